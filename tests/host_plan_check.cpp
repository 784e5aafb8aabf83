// host_plan_check.cpp -- CPU checks of the host-side index arithmetic of the tile kernels, built by
// tests/test_host_plan_cpu.py with g++ -fsanitize=address,undefined (no HIP, no GPU):
//   * TileMap: over ids 0 .. items()-1, tile() yields every (tile row, tile column, k-split) of the
//     problem exactly once and nothing outside it, for every block shape and walk order;
//   * the same for the "live rows" rebuild that k_dhidden makes from a device-side token count;
//   * make_plan: workspace regions are 256-byte aligned, do not overlap, end inside the totals;
//     the vocab splits of the d_hidden product cover V; chunks cover N;
//   * the no-alloc chunk search returns the largest chunk that fits, or refuses;
//   * the sampler's work items cover the vocabulary.
// Prints "ok <checks>" and exits 0, or a message and exits 1.
#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "../mllm-jax_amd/csrc/plan.hpp"
#include "../mllm-jax_amd/csrc/tile_map.hpp"

using mj::TileMap;
using namespace mj::host;

static long g_checks = 0;
#define CHECK(cond, ...)                                   \
  do {                                                     \
    ++g_checks;                                            \
    if (!(cond)) {                                         \
      std::fprintf(stderr, "FAILED %s:%d: %s\n  ", __FILE__, __LINE__, #cond); \
      std::fprintf(stderr, __VA_ARGS__);                   \
      std::fprintf(stderr, "\n");                          \
      std::exit(1);                                        \
    }                                                      \
  } while (0)

static void check_bijection(const TileMap& m, const char* what) {
  const int tm = m.tiles_m, tn = m.tiles_n, sp = m.splits;
  std::vector<unsigned char> seen((size_t)tm * tn * sp, 0);
  const int items = m.items();
  CHECK(items % 256 == 0 && items >= 0, "%s: items %d", what, items);
  long hits = 0;
  for (int id = 0; id < items; ++id) {
    int a = -1, b = -1, s = -1;
    if (!m.tile(id, a, b, s)) continue;
    CHECK(a >= 0 && a < tm && b >= 0 && b < tn && s >= 0 && s < sp, "%s: id %d -> (%d, %d, %d) outside %d x %d x %d",
          what, id, a, b, s, tm, tn, sp);
    unsigned char& cell = seen[((size_t)s * tm + a) * tn + b];
    CHECK(cell == 0, "%s: (%d, %d, %d) produced twice (id %d)", what, a, b, s, id);
    cell = 1;
    ++hits;
  }
  CHECK(hits == (long)tm * tn * sp, "%s: %ld of %ld tiles produced (tm %d tn %d splits %d lgm %d lgs %d n_first %d)",
        what, hits, (long)tm * tn * sp, tm, tn, sp, m.lgm, m.lgs, m.n_first);
  // ids past the end never yield a tile
  for (int id = items; id < items + 512; ++id) {
    int a, b, s;
    CHECK(!m.tile(id, a, b, s), "%s: id %d past items() yields a tile", what, id);
  }
}

static void tile_map_sweep() {
  const int dims[] = {0, 1, 2, 3, 4, 5, 8, 9, 14, 16, 33, 64, 129, 594};
  const int splits[] = {1, 2, 3, 7, 32};
  for (int tm : dims)
    for (int tn : dims) {
      if ((long)tm * tn > 20000) continue;
      for (int sp : splits)
        for (int nf = 0; nf < 2; ++nf) {
          if ((long)tm * tn * sp <= 30000)
            for (int ls = 0; ls <= 5; ++ls)
              for (int lm = 0; lm + ls <= 5; ++lm) check_bijection(TileMap(tm, tn, nf, lm, sp, ls), "explicit shape");
          const TileMap picked = TileMap::pick_shape(tm, tn, nf, sp);
          CHECK(picked.lgm + picked.lgn + picked.lgs == 5 && picked.lgm >= 0 && picked.lgn >= 0 && picked.lgs >= 0,
                "pick_shape exponents %d %d %d", picked.lgm, picked.lgn, picked.lgs);
          check_bijection(picked, "pick_shape");
          // k_dhidden rebuilds the list for the live rows of tiles (0 .. tm) with the launch's shape; the
          // launch has items() of the full list, which must cover the rebuilt one
          for (int live = 0; live <= tm; live += (tm > 8 ? tm / 4 + 1 : 1)) {
            const TileMap lv(live, picked.tiles_n, picked.n_first, picked.lgm, picked.splits, picked.lgs);
            check_bijection(lv, "live rebuild");
            CHECK(lv.items() <= picked.items(), "live list longer than the launch: %d > %d", lv.items(), picked.items());
          }
        }
    }
}

static MjGrpoDesc desc(int64_t n, int64_t h, int64_t v, int64_t chunk = 0, uint32_t flags = 0, float temp = 1.f,
                       uint32_t splits = 0) {
  MjGrpoDesc d;
  std::memset(&d, 0, sizeof d);
  d.n_tokens = n; d.hidden = h; d.vocab = v; d.ld_hidden = h; d.ld_w = v; d.chunk_tokens = chunk;
  d.temperature = temp; d.inv_total_valid_tokens = 1.f; d.grad_loss_scale = 1.f; d.flags = flags;
  d.dhidden_splits = splits;
  return d;
}

struct Region { size_t at, bytes; const char* name; };

static void check_plan(const MjGrpoDesc& d, bool launches = true) {
  Plan p;
  const int rc = make_plan(&d, &p);
  CHECK(rc == MJ_GRPO_OK, "make_plan(%lld, %lld, %lld, chunk %lld): %s", (long long)d.n_tokens, (long long)d.hidden,
        (long long)d.vocab, (long long)d.chunk_tokens, g_err);
  CHECK(p.chunk >= 1 && p.chunk <= p.N && p.n_pad % 256 == 0 && p.n_pad >= p.chunk && p.n_pad - p.chunk < 256,
        "chunk %lld n_pad %lld", (long long)p.chunk, (long long)p.n_pad);
  CHECK(p.chunk == p.N || p.chunk % 256 == 0, "a chunk that is not the whole batch is a multiple of 256");
  CHECK(p.parts == 2 * ((p.V + 255) / 256), "parts");
  CHECK(p.dh_splits >= 1 && p.dh_splits <= 32, "splits %d", p.dh_splits);
  CHECK(p.dh_k_per_split % 64 == 0 && p.dh_k_per_split * p.dh_splits >= p.V, "k_per_split %lld x %d < V %lld",
        (long long)p.dh_k_per_split, p.dh_splits, (long long)p.V);
  CHECK(p.dh_k_per_split * (p.dh_splits - 1) < p.V || p.dh_splits == 1, "an empty vocab split: %lld x %d, V %lld",
        (long long)p.dh_k_per_split, p.dh_splits, (long long)p.V);
  const size_t n4 = (size_t)p.N * 4, np4 = (size_t)p.n_pad * 4, stats = (size_t)p.parts * p.n_pad * 4;
  std::vector<Region> r = {
      {p.zy, n4, "zy"}, {p.term, n4, "term"}, {p.eterm, n4, "eterm"}, {p.pm, stats, "pm"}, {p.pl, stats, "pl"},
      {p.ps, stats, "ps"}, {p.plt, d.temperature != 1.f ? stats : 0, "plt"}, {p.g, np4, "g"}, {p.ge, np4, "ge"},
      {p.hent, np4, "hent"}, {p.state, 256, "state"}};
  if (p.compact) {
    r.push_back({p.perm, n4, "perm"});
    r.push_back({p.n_live, 256, "n_live"});
    r.push_back({p.hid_p, (size_t)p.N * p.H * 2, "hid_p"});
    r.push_back({p.tgt_p, n4, "tgt_p"});
    for (size_t f : p.fin_p) r.push_back({f, n4, "fin_p"});
    for (size_t f : p.fout_p) r.push_back({f, n4, "fout_p"});
  }
  const size_t fwd_regions = r.size();
  r.push_back({p.dh_p, p.compact ? (size_t)p.N * p.H * 2 : 0, "dh_p"});
  r.push_back({p.rs, np4, "rs"});
  r.push_back({p.dead, (size_t)p.n_pad / 8, "dead"});
  r.push_back({p.hs, (size_t)p.n_pad * p.H * 2, "hs"});
  r.push_back({p.zt, (size_t)p.n_pad * p.ld_z * 2, "zt"});
  r.push_back({p.part, p.dh_splits > 1 ? (size_t)p.dh_splits * p.n_pad * p.H * 4 : 0, "part"});
  const size_t bwd_regions = r.size();
  const size_t vblocks = (size_t)((p.N + kValueRows - 1) / kValueRows);
  r.push_back({p.v_term, n4, "v_term"});
  r.push_back({p.v_dv, (size_t)rup(p.N, 256) * 4, "v_dv"});
  r.push_back({p.v_dv_p, p.compact ? (size_t)rup(p.N, 256) * 4 : 0, "v_dv_p"});
  r.push_back({p.v_part, vblocks * p.H * 4, "v_part"});
  size_t end = 0;
  for (size_t i = 0; i < r.size(); ++i) {
    CHECK(r[i].at % 256 == 0, "%s not 256-byte aligned", r[i].name);
    CHECK(r[i].at >= end, "%s starts at %zu inside the region before it (ends %zu)", r[i].name, r[i].at, end);
    end = r[i].at + r[i].bytes;
    const size_t total = i < fwd_regions ? p.total_fwd : (i < bwd_regions ? p.total_bwd : p.total_value);
    CHECK(end <= total, "%s ends at %zu past its total %zu", r[i].name, end, total);
  }
  CHECK(p.total_fwd <= p.total_bwd && p.total_bwd <= p.total_value, "totals not nested");
  // the dead-token words: k_finalize writes n_pad / 16 16-bit pieces, the loaders read n_pad / 64 words
  CHECK((size_t)p.n_pad / 16 * 2 == (size_t)p.n_pad / 8 && (size_t)p.n_pad / 64 * 8 == (size_t)p.n_pad / 8, "dead bits");
  // chunks cover N; every chunk's padded row count fits the buffers sized for n_pad
  int64_t covered = 0;
  for (int64_t c0 = 0; c0 < p.N; c0 += p.chunk) {
    const int64_t nc = std::min(p.chunk, p.N - c0);
    CHECK(rup(nc, 256) <= p.n_pad, "chunk at %lld: %lld rows padded past n_pad", (long long)c0, (long long)nc);
    covered += nc;
    // the launches of this chunk: every tile of each product exactly once (spot check at the real shapes)
    if (launches && p.V <= 160000 && p.H <= 4096 && nc <= 32768 && (c0 == 0 || c0 + nc == p.N)) {
      check_bijection(TileMap::pick_shape((int)((p.V + 255) / 256), (int)((nc + 255) / 256), 1, 1), "logits launch");
      check_bijection(TileMap::pick_shape((int)((nc + 255) / 256), (int)((p.H + 255) / 256), 0, p.dh_splits), "d_hidden launch");
      check_bijection(TileMap::pick_shape((int)((p.V + 255) / 256), (int)((p.H + 255) / 256), 0, 1), "d_w launch");
    }
  }
  CHECK(covered == p.N, "chunks cover %lld of %lld tokens", (long long)covered, (long long)p.N);
}

static void plan_sweep() {
  const int64_t ns[] = {1, 17, 255, 256, 257, 512, 4096, 16384, 16385, 32768, 100000};
  const int64_t hs[] = {8, 64, 896, 1536, 2304, 3584, 4096};
  const int64_t vs[] = {8, 296, 2048, 128256, 151936, 152064, 256000};
  const int64_t chunks[] = {0, 1, 256, 300, 2048, 8192, 16384, 1 << 20};
  for (int64_t n : ns)
    for (int64_t h : hs)
      for (int64_t v : vs)
        for (int64_t c : chunks)
          for (uint32_t flags : {0u, (uint32_t)MJ_GRPO_FLAG_SKIP_MASKED, (uint32_t)(MJ_GRPO_FLAG_SFT | MJ_GRPO_FLAG_DW_BF16)})
            for (float t : {1.f, 0.7f})
              for (uint32_t sp : {0u, 1u, 5u, 32u})
                check_plan(desc(n, h, v, c, flags, t, sp), flags == 0 && t == 1.f && (sp == 0 || sp == 5) && (h % 512 == 0 || h == 896));
  // pick_splits: whole rounds of 256 workgroups, at most 32 pieces
  for (int64_t tiles = 1; tiles <= 4096; ++tiles) {
    const int s = pick_splits(tiles);
    CHECK(s >= 1 && s <= 32, "pick_splits(%lld) = %d", (long long)tiles, s);
  }
  // rejected descriptors come back as a status and a message, without touching anything
  Plan p;
  MjGrpoDesc bad = desc(0, 64, 512);
  CHECK(make_plan(&bad, &p) == MJ_GRPO_ERR_SHAPE && std::strlen(g_err) > 10, "n = 0 accepted");
  bad = desc(64, 60, 512);
  CHECK(make_plan(&bad, &p) == MJ_GRPO_ERR_ALIGN, "hidden not a multiple of 8 accepted");
  bad = desc(64, 64, 512, 0, 1u << 9);
  CHECK(make_plan(&bad, &p) == MJ_GRPO_ERR_UNSUPPORTED, "unknown flag accepted");
  CHECK(make_plan(nullptr, &p) == MJ_GRPO_ERR_NULL, "null descriptor accepted");
}

static void noalloc_sweep() {
  const size_t scratch = (size_t)MJ_GRPO_NOALLOC_SCRATCH_BYTES;
  const int64_t ns[] = {1, 300, 2048, 4096, 16384, 100000, 2000000};
  const int64_t vs[] = {512, 32000, 152064, 256000, 1 << 21};
  for (int64_t n : ns)
    for (int64_t v : vs) {
      MjGrpoDesc d = desc(n, 64, v), out;
      Plan p;
      const int rc = noalloc_plan(&d, scratch, &out, &p);
      if (rc != MJ_GRPO_OK) {
        CHECK(rc == MJ_GRPO_ERR_WORKSPACE, "no-alloc plan: status %d (%s)", rc, g_err);
        // refused: not even 256-token chunks fit
        MjGrpoDesc small = d;
        small.chunk_tokens = 256;
        Plan q;
        CHECK(make_plan(&small, &q) == MJ_GRPO_OK && q.total_fwd > scratch, "refused although 256-token chunks fit");
        continue;
      }
      CHECK(p.total_fwd <= scratch, "no-alloc plan of %zu bytes past the array", p.total_fwd);
      CHECK(out.chunk_tokens >= 256 && out.chunk_tokens % 256 == 0 && out.chunk_tokens <= 16384, "chunk %lld",
            (long long)out.chunk_tokens);
      // the next larger chunk does not fit (or the batch / the 16384 cap ends the search)
      if (out.chunk_tokens < 16384 && out.chunk_tokens < rup(n, 256)) {
        MjGrpoDesc next = d;
        next.chunk_tokens = out.chunk_tokens + 256;
        Plan q;
        CHECK(make_plan(&next, &q) == MJ_GRPO_OK && q.total_fwd > scratch, "a larger chunk (%lld) would have fitted",
              (long long)next.chunk_tokens);
      }
      check_plan(out);
    }
  MjGrpoDesc d = desc(4096, 64, 152064, 16384), out;
  Plan p;
  CHECK(noalloc_plan(&d, scratch, &out, &p) == MJ_GRPO_ERR_WORKSPACE, "an explicit chunk that does not fit was accepted");
}

static void sampler_sweep() {
  for (int64_t b : {1, 8, 64, 128, 129, 192, 256, 1000})
    for (int64_t v : {8, 512, 32000, 152064, 256000, 1 << 21}) {
      int bn;
      int64_t tiles_n, rows;
      sample_tiles(b, v, &bn, &tiles_n, &rows);
      CHECK((bn == 128 || bn == 256) && tiles_n * bn >= b && (tiles_n - 1) * bn < b, "batch tiles: bn %d x %lld for %lld",
            bn, (long long)tiles_n, (long long)b);
      CHECK(rows >= 8 && rows <= 256 && rows % 8 == 0, "tile_rows %lld", (long long)rows);
      const int64_t items = (v + rows - 1) / rows;
      CHECK(items * rows >= v && (items - 1) * rows < v, "vocab items");
      check_bijection(TileMap::pick_shape((int)items, (int)tiles_n, 1, 1), "sampler launch");
    }
}

int main() {
  tile_map_sweep();
  plan_sweep();
  noalloc_sweep();
  sampler_sweep();
  std::printf("ok %ld\n", g_checks);
  return 0;
}
