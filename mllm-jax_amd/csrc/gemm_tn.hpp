// gemm_tn.hpp -- bf16 MFMA tile engine for gfx950 (CDNA4), wave64.
//
// C[M,N] (fp32 accumulators) = A[M,K] * B[N,K]^T, both operands K-contiguous ("TN").
// One workgroup of 256 threads (4 wavefronts, 2x2) owns a BM x BN tile; each wavefront owns
// (BM/2) x (BN/2) as a grid of 32x32 MFMA blocks (v_mfma_f32_32x32x16_bf16).
//
// K is walked in slices of 32 through a ring of LDS stages.  Global memory is copied straight
// into LDS (buffer_load_dwordx4 ... lds: no staging registers, no ds_write), several slices
// ahead of the MFMAs, so the load latency is covered by (STAGES-1) slices of math.  Rows past the
// operand's end read as zero through the buffer descriptor's range check; K tails are masked
// per 16-byte chunk.  The LDS image of a slice is 64 bytes per row; the 16-byte chunk a lane
// fetches is XOR-permuted within its row so that the ds_read_b128 of 16 consecutive rows hits 16
// different bank groups.
//
// The three contractions of the loss path are instances of this engine with different epilogues:
//   logits^T[V,n] = Wt[V,H] * hidden[n,H]^T      (online-softmax statistics epilogue)
//   dHidden[n,H]  = dZ[n,V] * W[H,V]^T
//   dW[H,V]       = hiddenT[H,n] * dZt[V,n]^T
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mj {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define MJ_DEV __device__ __forceinline__

constexpr int kThreads = 256;
constexpr int kBK = 32;              // K elements per LDS stage
constexpr int kRowBytes = kBK * 2;   // 64 bytes per tile row in LDS
constexpr uint32_t kOob = 0x7ffffff0u;   // byte offset that every descriptor below rejects

typedef __attribute__((address_space(3))) void* lds_ptr_t;

MJ_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  // raw buffer (stride 0), 32-bit data format word for gfx9-class descriptors
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// s_waitcnt with only the vector-memory counter constrained (gfx9 encoding: vmcnt = [15:14|3:0]).
template <int N>
MJ_DEV void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt is 6 bits");
  __builtin_amdgcn_s_waitcnt(0x0f70 | (N & 15) | ((N >> 4) << 14));
}
MJ_DEV void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xc07f); }

// Position of 16-byte chunk c of tile row r inside the row's 64 bytes.
MJ_DEV int swz(int r) { return ((r >> 1) & 3) ^ ((r >> 3) & 1); }

// Maps a linear workgroup id to a tile so that (a) the 32 workgroups that land on one
// XCD at a time (ids congruent mod 8 go to the same XCD) form a GM x GN block of tiles
// sharing operand slices in that XCD's L2, and (b) consecutive blocks walk along M first.
template <int GM, int GN>
struct TileMap {
  int tiles_m, tiles_n, sb_m, sb_n;
  __host__ __device__ TileMap(int tm, int tn)
      : tiles_m(tm), tiles_n(tn), sb_m((tm + GM - 1) / GM), sb_n((tn + GN - 1) / GN) {}
  __host__ int grid() const {
    int sb = sb_m * sb_n;
    return ((sb + 7) / 8) * 8 * (GM * GN);
  }
  MJ_DEV bool tile(int pid, int& tm, int& tn) const {
    const int xcd = pid & 7, q = pid >> 3;
    const int sb = (q / (GM * GN)) * 8 + xcd, within = q % (GM * GN);
    if (sb >= sb_m * sb_n) return false;
    tm = (sb % sb_m) * GM + within % GM;
    tn = (sb / sb_m) * GN + within / GM;
    return tm < tiles_m && tn < tiles_n;
  }
};

template <int BM, int BN, int STAGES = 4>
struct GemmTN {
  static_assert(BM % 64 == 0 && BN % 64 == 0, "tile sides are multiples of 64");
  static constexpr int WM = BM / 2, WN = BN / 2;     // wavefront tile
  static constexpr int MI = WM / 32, NI = WN / 32;   // 32x32 blocks per wavefront
  static constexpr int A_LD = BM / 64, B_LD = BN / 64;   // 16-byte loads per thread per stage
  static constexpr int LPS = A_LD + B_LD;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int kLdsBytes = STAGES * kStageBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS is 160 KB per CU");
  static_assert((STAGES - 1) * LPS < 64, "outstanding loads must fit the vmcnt counter");

  // acc[mi][ni][r]: row = mi*32 + (r/4)*8 + (lane/32)*4 + r%4, col = ni*32 + lane%32
  // within the wavefront tile whose origin is (wm*WM, wn*WN).
  f32x16 acc[MI][NI];

  // A: tile origin pointer (row m0, k 0), rows_a valid rows, lda elements; same for B.
  MJ_DEV void run(const __bf16* A, int rows_a, int64_t lda, const __bf16* B, int rows_b,
                  int64_t ldb, int K, char* smem) {
    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    const int l31 = lane & 31, lhi = lane >> 5;

    const uint32_t bytes_a = (uint32_t)min((int64_t)min(rows_a, BM) * lda * 2, (int64_t)0x7fffff00);
    const uint32_t bytes_b = (uint32_t)min((int64_t)min(rows_b, BN) * ldb * 2, (int64_t)0x7fffff00);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A, bytes_a);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(B, bytes_b);

    // Direct-to-LDS copy: one instruction of one wavefront fills 1024 contiguous LDS bytes
    // (16 tile rows), lane -> (row = lane/4, slot = lane%4); the lane fetches global chunk
    // slot ^ swz(row) so the LDS image is the swizzled one.
    const int ld_row = wave * 16 + (lane >> 2);              // + 64*i
    const int ld_chunk = (lane & 3) ^ swz(lane >> 2);        // row base is a multiple of 16
    uint32_t goff_a[A_LD], goff_b[B_LD];
#pragma unroll
    for (int i = 0; i < A_LD; ++i) goff_a[i] = (uint32_t)((ld_row + 64 * i) * lda * 2 + ld_chunk * 16);
#pragma unroll
    for (int i = 0; i < B_LD; ++i) goff_b[i] = (uint32_t)((ld_row + 64 * i) * ldb * 2 + ld_chunk * 16);
    const int klimit = K - ld_chunk * 8;   // chunk is inside the row iff k0 < klimit

    auto issue = [&](int slice) {
      const int k0 = slice * kBK;
      char* base = smem + (slice % STAGES) * kStageBytes + wave * 1024;
      if (k0 + kBK <= K) {
#pragma unroll
        for (int i = 0; i < A_LD; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + i * 4096), 16, goff_a[i], k0 * 2, 0, 0);
#pragma unroll
        for (int i = 0; i < B_LD; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(base + BM * kRowBytes + i * 4096), 16,
                                                   goff_b[i], k0 * 2, 0, 0);
      } else {   // K tail (or past the end): chunks at or beyond K read as zero
        const bool in = k0 < klimit;
#pragma unroll
        for (int i = 0; i < A_LD; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(base + i * 4096), 16,
                                                   in ? goff_a[i] + k0 * 2 : kOob, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < B_LD; ++i)
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rb, (lds_ptr_t)(base + BM * kRowBytes + i * 4096), 16,
                                                   in ? goff_b[i] + k0 * 2 : kOob, 0, 0, 0);
      }
    };

    // LDS read positions: row within a 32-row block = lane % 32, k-chunk = 2*ks + lane/32
    int rd_off[2];
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) rd_off[ks] = l31 * kRowBytes + (((2 * ks + lhi) ^ swz(l31)) << 4);
    const int a_base = wm * WM * kRowBytes;
    const int b_base = BM * kRowBytes + wn * WN * kRowBytes;

    bf16x8 fa[2][MI], fb[2][NI];
    auto read_frags = [&](int slice, int ks, int buf) {
      const char* sbase = smem + (slice % STAGES) * kStageBytes;
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
        fa[buf][mi] = *(const bf16x8*)(sbase + a_base + mi * 32 * kRowBytes + rd_off[ks]);
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
        fb[buf][ni] = *(const bf16x8*)(sbase + b_base + ni * 32 * kRowBytes + rd_off[ks]);
    };
    auto mma = [&](int buf) {
#pragma unroll
      for (int mi = 0; mi < MI; ++mi)
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
          acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][mi], fb[buf][ni], acc[mi][ni], 0, 0, 0);
    };

#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    const int KT = (K + kBK - 1) / kBK;
#pragma unroll
    for (int s = 0; s < STAGES - 1; ++s) issue(s);
    wait_vmcnt<(STAGES - 2) * LPS>();   // slice 0 has landed (this wavefront's part)
    __builtin_amdgcn_s_barrier();       // ... and everyone else's
    read_frags(0, 0, 0);
    for (int kt = 0; kt < KT; ++kt) {
      issue(kt + STAGES - 1);           // into the stage that slice kt-1 occupied
      read_frags(kt, 1, 1);
      mma(0);
      wait_lgkmcnt0();                  // this wavefront is done reading slice kt
      wait_vmcnt<(STAGES - 2) * LPS>(); // slice kt+1 has landed
      __builtin_amdgcn_s_barrier();
      read_frags(kt + 1, 0, 0);
      mma(1);
    }
    wait_vmcnt<0>();                    // drain the (empty) prefetches before LDS is reused
  }
};

}  // namespace mj
