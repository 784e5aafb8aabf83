// gemm_tn.hpp -- bf16 MFMA tile engine for gfx950 (CDNA4), wave64.
//
// C[M,N] (fp32 accumulators) = A[M,K] * B[N,K]^T, both operands K-contiguous
// ("TN").  One workgroup of 256 threads (4 wavefronts, 2x2) owns a BM x BN tile;
// each wavefront owns (BM/2) x (BN/2) as a grid of 32x32 MFMA blocks
// (v_mfma_f32_32x32x16_bf16).  K is walked in slices of 64: global -> registers
// (16-byte buffer loads, out-of-range rows / K tails read as zero through the
// buffer descriptor) -> LDS (XOR-swizzled 16-byte chunks, two stages) -> MFMA.
//
// The three contractions of the loss path are instances of this engine with
// different epilogues:
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
constexpr int kBK = 64;              // K elements per LDS stage
constexpr int kRowBytes = kBK * 2;   // 128 bytes per tile row in LDS

MJ_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  // raw buffer (stride 0), 32-bit data format word for gfx9-class descriptors
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

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

template <int BM, int BN>
struct GemmTN {
  static constexpr int WM = BM / 2, WN = BN / 2;     // wavefront tile
  static constexpr int MI = WM / 32, NI = WN / 32;   // 32x32 blocks per wavefront
  static constexpr int A_LD = BM * 8 / kThreads;     // 16-byte loads per thread per stage
  static constexpr int B_LD = BN * 8 / kThreads;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;

  // acc[mi][ni][r]: row = mi*32 + (r/4)*8 + (lane/32)*4 + r%4, col = ni*32 + lane%32
  // within the wavefront tile whose origin is (wm*WM, wn*WN).
  f32x16 acc[MI][NI];

  // A: tile origin pointer (row m0, k 0), rows_a valid rows, lda elements; same for B.
  MJ_DEV void run(const __bf16* A, int rows_a, int64_t lda, const __bf16* B, int rows_b,
                  int64_t ldb, int K, char* smem) {
    const int t = threadIdx.x;
    const int lane = t & 63, wave = t >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    const int lrow = t >> 3, lchunk = t & 7;

    const uint32_t bytes_a = (uint32_t)min((int64_t)min(rows_a, BM) * lda * 2, (int64_t)0x7ffffff0);
    const uint32_t bytes_b = (uint32_t)min((int64_t)min(rows_b, BN) * ldb * 2, (int64_t)0x7ffffff0);
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(A, bytes_a);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(B, bytes_b);

    uint32_t goff_a[A_LD], goff_b[B_LD];
#pragma unroll
    for (int i = 0; i < A_LD; ++i) goff_a[i] = (uint32_t)((lrow + 32 * i) * lda * 2 + lchunk * 16);
#pragma unroll
    for (int i = 0; i < B_LD; ++i) goff_b[i] = (uint32_t)((lrow + 32 * i) * ldb * 2 + lchunk * 16);

    // LDS write position of this thread's chunk (row & 7 == lrow & 7 for every i)
    const int st_off = lrow * kRowBytes + ((lchunk ^ (lrow & 7)) << 4);
    // LDS read positions: row within a 32-row block = lane % 32, chunk = 2*ks + lane/32
    const int l31 = lane & 31, lhi = lane >> 5;
    int rd_off[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) rd_off[ks] = l31 * kRowBytes + (((2 * ks + lhi) ^ (lane & 7)) << 4);
    const int a_base = wm * WM * kRowBytes;
    const int b_base = BM * kRowBytes + wn * WN * kRowBytes;

#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    u32x4 sa[A_LD], sb[B_LD];
    auto gload = [&](int k0) {
      const bool kin = (k0 + lchunk * 8) < K;
      const uint32_t kb = (uint32_t)k0 * 2;
#pragma unroll
      for (int i = 0; i < A_LD; ++i)
        sa[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, kin ? goff_a[i] + kb : 0x7ffffff0u, 0, 0);
#pragma unroll
      for (int i = 0; i < B_LD; ++i)
        sb[i] = __builtin_amdgcn_raw_buffer_load_b128(rb, kin ? goff_b[i] + kb : 0x7ffffff0u, 0, 0);
    };
    auto lstore = [&](int stage) {
      char* base = smem + stage * kStageBytes + st_off;
#pragma unroll
      for (int i = 0; i < A_LD; ++i) *(u32x4*)(base + i * 32 * kRowBytes) = sa[i];
#pragma unroll
      for (int i = 0; i < B_LD; ++i) *(u32x4*)(base + BM * kRowBytes + i * 32 * kRowBytes) = sb[i];
    };

    const int KT = (K + kBK - 1) / kBK;
    gload(0);
    lstore(0);
    __syncthreads();
    for (int kt = 0; kt < KT; ++kt) {
      gload((kt + 1) * kBK);   // past the end: every lane predicated to the zero-reading offset
      const char* sbase = smem + (kt & 1) * kStageBytes;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        bf16x8 a[MI], b[NI];
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
          a[mi] = *(const bf16x8*)(sbase + a_base + mi * 32 * kRowBytes + rd_off[ks]);
#pragma unroll
        for (int ni = 0; ni < NI; ++ni)
          b[ni] = *(const bf16x8*)(sbase + b_base + ni * 32 * kRowBytes + rd_off[ks]);
#pragma unroll
        for (int mi = 0; mi < MI; ++mi)
#pragma unroll
          for (int ni = 0; ni < NI; ++ni)
            acc[mi][ni] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[mi], b[ni], acc[mi][ni], 0, 0, 0);
      }
      lstore((kt + 1) & 1);
      __syncthreads();
    }
  }
};

}  // namespace mj
