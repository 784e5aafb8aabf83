// gemm_tn.hpp -- bf16 MFMA tile engine for gfx950 (CDNA4), wave64.
//
// C[M,N] (fp32 accumulators) = A[M,K] * B[N,K]^T, both operands K-contiguous ("TN").
// One workgroup of 256 threads (4 wavefronts, 2x2) owns a BM x BN tile; each wavefront owns
// (BM/2) x (BN/2) as a grid of 32x32 MFMA blocks (v_mfma_f32_32x32x16_bf16).
//
// K is walked in slices of 64 through two LDS stages.  A slice travels global memory ->
// registers (16-byte buffer loads, every 8 lanes cover one full 128-byte line of a tile row) ->
// LDS (ds_write_b128) -> MFMA operands (ds_read_b128).  The loads of slice k+2 and the LDS writes
// of slice k+1 are issued one at a time between the MFMAs of slice k, so the texture-address unit
// sees an even trickle instead of a burst and every load has a whole slice of math to land.  Rows
// past the operand's end read as zero through the buffer descriptor's range check; K tails are
// masked per 16-byte chunk.  The LDS image of a slice is 128 bytes per row; 16-byte chunk c of
// row r sits at slot c ^ swz(r), which keeps both the writes and the ds_read_b128 of consecutive
// rows bank-conflict free whether the LDS serves 8 or 16 lanes per clock.  MFMA operands are
// double-buffered in registers: the LDS reads of k-step s+1 sit between the MFMAs of k-step s.
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
constexpr int kBK = 64;              // K elements per LDS stage
constexpr int kRowBytes = kBK * 2;   // 128 bytes per tile row in LDS
constexpr int kSteps = kBK / 16;     // MFMA k-steps per stage
constexpr uint32_t kOob = 0x7ffffff0u;   // byte offset that every descriptor below rejects

MJ_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  // raw buffer (stride 0), 32-bit data format word for gfx9-class descriptors
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// s_waitcnt with only the LDS/scalar counter constrained (gfx9 encoding).
MJ_DEV void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xc07f); }

// Chunk c of tile row r lives at 16-byte slot c ^ swz(r) of the row's 128 bytes.
MJ_DEV int swz(int r) { return (r ^ (r >> 3)) & 7; }

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
  static_assert(BM % 32 == 0 && BN % 32 == 0, "tile sides are multiples of 32");
  static constexpr int WM = BM / 2, WN = BN / 2;     // wavefront tile
  static constexpr int MI = WM / 32, NI = WN / 32;   // 32x32 blocks per wavefront
  static constexpr int A_LD = BM / 32, B_LD = BN / 32;   // 16-byte loads per thread per stage
  static constexpr int LPS = A_LD + B_LD;
  static constexpr int kStageBytes = (BM + BN) * kRowBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS is 160 KB per CU");

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

    // Global -> register staging: thread t fetches chunk t%8 of tile rows t/8 + 32*i.
    const int ld_row = t >> 3, ld_chunk = t & 7;
    uint32_t goff_a[A_LD], goff_b[B_LD];
#pragma unroll
    for (int i = 0; i < A_LD; ++i) goff_a[i] = (uint32_t)((ld_row + 32 * i) * lda * 2 + ld_chunk * 16);
#pragma unroll
    for (int i = 0; i < B_LD; ++i) goff_b[i] = (uint32_t)((ld_row + 32 * i) * ldb * 2 + ld_chunk * 16);
    const int klimit = K - ld_chunk * 8;   // chunk is inside the row iff k0 < klimit
    // swz(row + 32*i) == swz(row): one LDS write offset serves every i
    const int st_off = ld_row * kRowBytes + ((ld_chunk ^ swz(ld_row)) << 4);

    u32x4 stage[LPS];
    // Load j (of the LPS this thread issues per slice).  Branch-free: a chunk at or beyond K
    // (K tail, or a whole slice past the end) is redirected to an offset the descriptor rejects.
    auto load_one = [&](int slice, int j) {
      const int k0 = slice * kBK;
      const bool in = k0 < klimit;
      if (j < A_LD)
        stage[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, in ? goff_a[j] : kOob, k0 * 2, 0);
      else
        stage[j] = __builtin_amdgcn_raw_buffer_load_b128(rb, in ? goff_b[j - A_LD] : kOob, k0 * 2, 0);
    };
    auto store_one = [&](int slice, int j) {
      char* base = smem + (slice & 1) * kStageBytes + st_off;
      if (j < A_LD)
        *(u32x4*)(base + j * 32 * kRowBytes) = stage[j];
      else
        *(u32x4*)(base + BM * kRowBytes + (j - A_LD) * 32 * kRowBytes) = stage[j];
    };

    // LDS read positions: row within a 32-row block = lane % 32, k-chunk = 2*ks + lane/32
    int rd_off[kSteps];
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) rd_off[ks] = l31 * kRowBytes + (((2 * ks + lhi) ^ swz(l31)) << 4);
    const int a_base = wm * WM * kRowBytes;
    const int b_base = BM * kRowBytes + wn * WN * kRowBytes;

    bf16x8 fa[2][MI], fb[2][NI];
    auto read_one = [&](int slice, int ks, int buf, int g) {   // fragment g of the MI + NI
      const char* sbase = smem + (slice & 1) * kStageBytes;
      if (g < MI)
        fa[buf][g] = *(const bf16x8*)(sbase + a_base + g * 32 * kRowBytes + rd_off[ks]);
      else
        fb[buf][g - MI] = *(const bf16x8*)(sbase + b_base + (g - MI) * 32 * kRowBytes + rd_off[ks]);
    };
    // One k-step, hand-scheduled: MI+NI groups, each = [LDS write of one staged chunk of the next
    // slice, then the global load that refills that staging register with the slice after it]
    // + one LDS read of the next k-step's fragments + this k-step's share of MFMAs.  The fences
    // keep the groups in this order, so the MFMA pipe always has work queued behind every memory
    // instruction.  `first` is the index of this k-step's first staged chunk (>= LPS: none left).
    constexpr int G = MI + NI, T = MI * NI;
    auto kstep = [&](int buf, int next_slice, int next_ks, int kt, int first) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        if (first + g < LPS) {
          store_one(kt + 1, first + g);
          load_one(kt + 2, first + g);
        }
        read_one(next_slice, next_ks, buf ^ 1, g);
#pragma unroll
        for (int p = g * T / G; p < (g + 1) * T / G; ++p)
          acc[p / NI][p % NI] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][p / NI], fb[buf][p % NI],
                                                                        acc[p / NI][p % NI], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    };

#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    static_assert(LPS <= 3 * G, "the staged chunks of a slice must fit the first three k-steps");
    const int KT = (K + kBK - 1) / kBK;
#pragma unroll
    for (int j = 0; j < LPS; ++j) load_one(0, j);
#pragma unroll
    for (int j = 0; j < LPS; ++j) {
      store_one(0, j);
      load_one(1, j);
    }
    wait_lgkmcnt0();
    __builtin_amdgcn_s_barrier();       // slice 0 is in LDS, slice 1 is on its way to the registers
#pragma unroll
    for (int g = 0; g < G; ++g) read_one(0, 0, 0, g);
    for (int kt = 0; kt < KT; ++kt) {
      // slice kt+1 moves registers -> the stage slice kt-1 occupied; slice kt+2 starts loading
      kstep(0, kt, 1, kt, 0);
      kstep(1, kt, 2, kt, G);
      kstep(0, kt, 3, kt, 2 * G);
      wait_lgkmcnt0();                  // own reads of slice kt and writes of slice kt+1 are done
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      kstep(1, kt + 1, 0, kt, LPS);
    }
  }
};

}  // namespace mj
