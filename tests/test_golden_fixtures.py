"""Golden fixtures (tests/golden/*.npz): the oracle must reproduce them on the CPU, and the HIP
path must match them on the GPU within the task's tolerances."""
import glob
import os

import numpy as np
import pytest

from oracle import grpo_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
FIXTURES = sorted(glob.glob(os.path.join(HERE, "golden", "*.npz")))


def _load(path):
    d = dict(np.load(path, allow_pickle=False))
    d["old_logps"] = d.get("old_logps")
    d["cap"] = float(d["softcap"]) or None
    return d


def test_fixtures_exist():
    assert len(FIXTURES) >= 4


@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[:-4])
def test_oracle_reproduces_fixture(path):
    d = _load(path)
    out = O.grpo_loss(d["hidden"], d["lm_head"], d["target_ids"], d["old_logps"], d["advantages"], d["mask"],
                      total_valid_token_count=float(d["total_valid_token_count"]),
                      epsilon_low=float(d["epsilon"][0]), epsilon_high=float(d["epsilon"][1]),
                      final_logit_softcap=d["cap"], seq_shape=tuple(int(x) for x in d["seq_shape"]))
    np.testing.assert_allclose(out["loss"], d["loss"], rtol=1e-12)
    np.testing.assert_allclose(out["per_token_logps"], d["per_token_logps"], atol=1e-12)
    np.testing.assert_allclose(out["token_entropy"], d["token_entropy"], atol=1e-12)
    np.testing.assert_allclose(out["d_hidden"], d["d_hidden"], atol=1e-7)
    np.testing.assert_allclose(out["d_lm_head"], d["d_lm_head"], atol=1e-7)


@pytest.mark.gpu
@pytest.mark.parametrize("path", FIXTURES, ids=lambda p: os.path.basename(p)[:-4])
def test_hip_path_matches_fixture(path):
    import torch
    import mllm_jax_amd as M
    d = _load(path)
    dev = torch.device("cuda:0")
    t = lambda x, dt=None: None if x is None else torch.as_tensor(x).to(dev if dt is None else dev, dtype=dt)
    met, (dh, dw) = M.grpo_loss_value_and_grad(
        t(d["hidden"], torch.bfloat16), t(d["lm_head"], torch.bfloat16), t(d["target_ids"]), t(d["old_logps"]),
        t(d["advantages"]), t(d["mask"]), total_valid_token_count=float(d["total_valid_token_count"]),
        epsilon_low=float(d["epsilon"][0]), epsilon_high=float(d["epsilon"][1]), final_logit_softcap=d["cap"],
        seq_shape=tuple(int(x) for x in d["seq_shape"]), return_token_entropy=True)
    torch.cuda.synchronize()
    rel = lambda a, b: np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30)
    assert np.abs(met["per_token_logps"].reshape(-1).cpu().numpy() - d["per_token_logps"]).max() <= 1e-3
    assert np.abs(met["token_entropy"].reshape(-1).cpu().numpy() - d["token_entropy"]).max() <= 1e-3
    assert abs(met["loss"].item() - d["loss"]) <= 1e-3 * abs(d["loss"]) + 1e-7
    assert rel(dh.float().cpu().numpy(), d["d_hidden"]) <= 2e-2
    assert rel(dw.cpu().numpy(), d["d_lm_head"]) <= 2e-2
    ok = np.isfinite(d["entropy"])
    assert np.abs(met["entropy"].cpu().numpy()[ok] - d["entropy"][ok]).max() <= 1e-3
