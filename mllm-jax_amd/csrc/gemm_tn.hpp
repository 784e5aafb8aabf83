// gemm_tn.hpp -- bf16 MFMA tile engine for gfx950 (CDNA4), wave64.
//
// C[M,N] (fp32 accumulators) = sum_k A(m,k) * B(n,k).  One workgroup of WAVES_M x WAVES_N
// wavefronts owns a BM x BN tile; each wavefront owns (BM/WAVES_M) x (BN/WAVES_N) as a grid of
// 32x32 MFMA blocks (v_mfma_f32_32x32x16_bf16; GemmTN) or of 16x16 blocks
// (v_mfma_f32_16x16x32_bf16 with the two k-steps of a block chained; GemmTN16, further down).
//
// Each operand may live in memory in either of two layouts, so a product can read its operands
// where they are:
//   kRowK : X[row][k], k contiguous  -- LDS image 128 bytes per tile row, MFMA fragments come
//           out with one ds_read_b128 per lane;
//   kKRow : X[k][row], rows contiguous -- LDS image 64 k-rows of 2*ROWS bytes, MFMA fragments
//           come out of two ds_read_b64_tr_b16 (the LDS transposing read of gfx950).
// Both give lane l of a fragment the same k order (8*(l/32) + 0..7), so they mix freely.
//
// K is walked in slices of 64 through two LDS stages.  A slice travels global memory ->
// registers (16-byte buffer loads that cover whole 128-byte lines) -> LDS (ds_write_b128) ->
// MFMA operands.  The loads of slice k+2 and the LDS writes of slice k+1 are issued one at a
// time between the MFMAs of slice k, so the texture-address unit and the LDS see an even
// trickle instead of bursts and every load has a whole slice of math to land.  Rows / k-rows
// past the operand's end read as zero through the buffer descriptor's range check; tails in
// the contiguous direction are masked per 16-byte chunk.  16-byte chunks are XOR-permuted
// inside their LDS row so that the writes and both kinds of fragment read are bank-conflict
// free.  MFMA operands are double-buffered in registers: the LDS reads of k-step s+1 sit
// between the MFMAs of k-step s.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "tile_map.hpp"

namespace mj {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(4))) short s16x4;
typedef __attribute__((ext_vector_type(8))) short s16x8;

#define MJ_DEV __device__ __forceinline__

constexpr int kThreads = 256;
constexpr int kBK = 64;              // K elements per LDS stage
constexpr int kSteps = kBK / 16;     // MFMA k-steps per stage
constexpr uint32_t kOob = 0x7ffffff0u;   // byte offset that every descriptor below rejects

enum Layout { kRowK = 0, kKRow = 1 };

MJ_DEV __amdgpu_buffer_rsrc_t make_rsrc(const void* p, int64_t bytes) {
  // raw buffer (stride 0), 32-bit data format word for gfx9-class descriptors
  const int64_t capped = bytes < 0 ? 0 : (bytes > 0x7fffff00 ? 0x7fffff00 : bytes);
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)capped, 0x00020000);
}

// Same, for descriptors built from per-wavefront (not per-workgroup) quantities: the pieces are
// pinned to scalar registers so that the memory instructions need no per-lane descriptor loop.
MJ_DEV __amdgpu_buffer_rsrc_t make_rsrc_wave(const void* p, int64_t bytes) {
  const uint64_t a = (uint64_t)p;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)a);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(a >> 32));
  const int64_t capped = bytes < 0 ? 0 : (bytes > 0x7fffff00 ? 0x7fffff00 : bytes);
  const int n = __builtin_amdgcn_readfirstlane((int)capped);
  return __builtin_amdgcn_make_buffer_rsrc((void*)(((uint64_t)hi << 32) | lo), 0, n, 0x00020000);
}

// s_waitcnt with only the LDS/scalar counter constrained (gfx9 encoding).
MJ_DEV void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xc07f); }

// One operand of the tile: ROWS tile rows (M or N direction) by 64 k per slice, 128*ROWS bytes of
// LDS per stage, ROWS*8/THREADS 16-byte chunks per thread per slice.
// DEAD: the caller knows which rows (kRowK) or k-rows (kKRow) of the operand are all zero and hands
// in a bit mask, one 64-bit word per 64 of them (bit set = zero, do not fetch).  Their loads get an
// offset that the descriptor rejects: the registers fill with zeros and no memory request is made.
// FRAG: rows per MFMA fragment, 32 (v_mfma_f32_32x32x16_bf16, GemmTN) or 16 (v_mfma_f32_16x16x32_bf16,
// GemmTN16); it selects the chunk permutation of the kRowK image.
template <int ROWS, int LAYOUT, int THREADS, bool DEAD = false, int FRAG = 32>
struct Operand {
  static constexpr int LD = ROWS * 8 / THREADS;
  static constexpr int RPP = THREADS / 8;          // kRowK: tile rows covered by one pass of the workgroup
  static constexpr int KPP = THREADS / (ROWS / 8); // kKRow: k-rows covered by one pass
  static constexpr int kBytes = ROWS * 128;

  const char* base;      // tile origin: (row 0, k 0)
  int64_t ld2;           // bytes between consecutive rows (kRowK) / k-rows (kKRow)
  int rows, K;           // valid rows of this tile, K extent
  __amdgpu_buffer_rsrc_t rsrc;   // kRowK: whole tile; kKRow: current slice (see slice_begin)
  uint32_t goff[LD];     // byte offset of this thread's chunk i inside the tile / slice
  int st_off;            // LDS byte offset of chunk 0 (kRowK) ...
  int st_off1;           // ... and of odd i for kKRow (bit 3 of the k-row enters the permutation)
  int klimit;            // kRowK: chunk is inside the row iff k0 < klimit
  bool col_ok;           // kKRow: this thread's chunk lies inside the valid rows
  int rd[4];             // LDS read offsets: kRowK per k-step, kKRow per fragment
  int rd16[LAYOUT == kRowK ? 4 : 8];   // 16-row fragments (GemmTN16): kRowK per (k-step of 32, fragment parity), kKRow per fragment

  // 64-byte segment permutation of the kKRow image: 8 k-rows read by one transposing read
  // ({r..r+3} and {r+8..r+11}) must land in 8 different segments of the 512-byte row.
  static MJ_DEV int sigma(int krow) { return (krow & 3) | ((krow >> 1) & 4); }
  // The k-major image for 16-row fragments.  One transposing read fetches, per 16-lane group g, the 32
  // bytes of the fragment's rows from the k-rows 8 g + 0..3: 16 k-rows at the same place of their 512
  // bytes, which all start in the same bank.  perm16 moves the 32-byte pairs of 16-byte chunks of a
  // k-row around (xor on chunk bits 1..4, a function of k-row bits 0, 1 and 3) so that the 16 pieces
  // of one read fall into different banks; found by timing all 65536 maps that are linear in k-row
  // bits 0, 1, 3, 4 on the GPU (a third of them are conflict free; the segment permutation above
  // costs 2.5 ns instead of 1.9 ns per read and CU with this access pattern).
  static MJ_DEV int perm16(int krow) { return ((krow & 1) * 12) ^ (((krow >> 1) & 1) * 6) ^ (((krow >> 3) & 1) * 5); }
  static MJ_DEV int kperm(int krow) { return FRAG == 16 ? (perm16(krow) << 1) : (sigma(krow) << 2); }
  // 16-byte chunk permutation of the kRowK image (see the file header); depends on r mod 32 only.
  // 32-row fragments (lane l reads row l % 32, chunk 2 ks + l / 32): r % 8 xor (r / 8) % 4.
  // 16-row fragments (lane l reads row l % 16, chunk 4 ks + l / 16) conflict under that permutation
  // (SQ_LDS_BANK_CONFLICT on every read, 3.4 ns instead of 2.6 ns per ds_read_b128 and CU).  Of the
  // 4096 permutations that are linear in the bits of r, timed one by one on the GPU, a third are
  // conflict free for both k-steps; this is one of them: bit 1 of r flips chunk bits 4, bit 2 flips
  // 3, bit 3 flips 6 (bit 0 needs nothing: odd rows start in the other half of the banks).
  static MJ_DEV int swz(int r) {
    if (FRAG == 32) return (r & 7) ^ ((r >> 3) & 3);
    return (((r >> 1) & 1) * 4) ^ (((r >> 2) & 1) * 3) ^ (((r >> 3) & 1) * 6);
  }

  // dead: kRowK -- the words covering this tile's ROWS rows (ROWS / 64 of them);
  //       kKRow -- the words of the K extent, one per slice ((K + 63) / 64 of them).
  MJ_DEV void init(const __bf16* p, int rows_valid, int64_t ld, int K_, int wave_row0, int t,
                   const uint64_t* dead = nullptr) {
    static_assert(LAYOUT == kRowK || ROWS == 256, "the k-major image is laid out for 256-row tiles");
    static_assert(!DEAD || (ROWS == 256 && THREADS == 256), "the dead-row masks assume 8 chunks per thread, 32 or 8 rows apart");
    const int lane = t & 63;
    base = (const char*)p;
    ld2 = ld * 2;
    rows = rows_valid < ROWS ? rows_valid : ROWS;
    K = K_;
    if (LAYOUT == kRowK) {
      const int row = t >> 3, chunk = t & 7;     // chunk t%8 of tile rows t/8 + RPP*i
      rsrc = make_rsrc(base, (int64_t)rows * ld2);
#pragma unroll
      for (int i = 0; i < LD; ++i) goff[i] = (uint32_t)((row + RPP * i) * ld2 + chunk * 16);
      if (DEAD) {
        // rows row + 32 i: bit row + 32 (i & 1) of word i / 2
#pragma unroll
        for (int i = 0; i < LD; ++i)
          if ((dead[i >> 1] >> (row + 32 * (i & 1))) & 1ull) goff[i] = kOob;
      }
      klimit = K - chunk * 8;
      st_off = row * 128 + ((chunk ^ swz(row)) << 4);   // swz(row + RPP*i) == swz(row)
      st_off1 = st_off;
      col_ok = true;
      const int l31 = lane & 31, lhi = lane >> 5;       // fragment row, k-chunk 2*ks + lane/32
#pragma unroll
      for (int ks = 0; ks < 4; ++ks)
        rd[ks] = (wave_row0 + l31) * 128 + (((2 * ks + lhi) ^ swz(l31)) << 4);
    } else {
      constexpr int CPR = ROWS / 8;              // 16-byte chunks per k-row
      const int krow = t / CPR, chunk = t % CPR; // chunk of k-rows krow + KPP*i
#pragma unroll
      for (int i = 0; i < LD; ++i) goff[i] = (uint32_t)((krow + KPP * i) * ld2 + chunk * 16);
      col_ok = chunk * 8 < rows;
      klimit = 0;
      st_off = krow * (ROWS * 2) + ((chunk ^ kperm(krow)) << 4);
      st_off1 = krow * (ROWS * 2) + ((chunk ^ kperm(krow + KPP)) << 4);   // differs only if KPP == 8
      // Transposing read: the 16 lanes of a group fetch 4 k-rows x 4 row-quads (8 bytes each) and
      // get back, lane i, the 4 k of row i.  Lane l: group g = l/16, s = l%16 reads k-row
      // (g/2)*8 + s/4 (+4 for the second read, +16*ks), quad (g%2)*4 + s%4 of the 32-row fragment.
      const int g = lane >> 4, s = lane & 15;
      const int kr = (g >> 1) * 8 + (s >> 2);
#pragma unroll
      for (int f = 0; f < 4; ++f) {
        const int quad = (wave_row0 + f * 32) / 4 + (g & 1) * 4 + (s & 3);
        rd[f] = kr * (ROWS * 2) + ((((quad >> 1) ^ (sigma(kr) << 2))) << 4) + (quad & 1) * 8;
      }
    }
  }

  // Read offsets for 16-row fragments of v_mfma_f32_16x16x32_bf16: lane l supplies row l % 16,
  // k = 8 (l / 16) + 0..7 of a 32-wide k-step.  kRowK: one 16-byte read at row (f * 16 + l % 16),
  // chunk 4 ks + l / 16; the chunk permutation depends on the row modulo 32, i.e. on f's parity.
  // kKRow: two transposing reads; lane l = 16 g + s addresses k-row 8 g + s / 4 (+ 4 for the second
  // read, + 32 ks), quad s % 4 of the fragment's four, and gets back the four k of row s.
  MJ_DEV void init16(int wave_row0, int t) {
    static_assert(FRAG == 16, "16-row fragments: the operand's image must be laid out for them");
    const int lane = t & 63, l15 = lane & 15, lq = lane >> 4;
    if (LAYOUT == kRowK) {
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int par = 0; par < 2; ++par)
          rd16[ks * 2 + par] = (wave_row0 + par * 16 + l15) * 128 + (((4 * ks + lq) ^ swz(par * 16 + l15)) << 4);
    } else {
      const int kr = 8 * lq + (l15 >> 2);
#pragma unroll
      for (int f = 0; f < 8; ++f) {
        const int quad = (wave_row0 + f * 16) / 4 + (l15 & 3);
        rd16[f] = kr * (ROWS * 2) + (((quad >> 1) ^ kperm(kr)) << 4) + (quad & 1) * 8;
      }
    }
  }
  MJ_DEV bf16x8 frag16(const char* stage, int f, int ks) const {
    if (LAYOUT == kRowK) return *(const bf16x8*)(stage + rd16[ks * 2 + (f & 1)] + (f >> 1) * 32 * 128);
    typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
    const char* p = stage + rd16[f] + ks * 32 * (ROWS * 2);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * (ROWS * 2)));
    const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, v);
  }

  // kKRow: point the descriptor at slice `slice` (its k-rows past K fall outside and read zero).
  MJ_DEV void slice_begin(int slice) {
    if (LAYOUT == kKRow) {
      const int k0 = slice * kBK;
      const int left = K - k0;
      rsrc = make_rsrc(base + (int64_t)k0 * ld2, (int64_t)(left < kBK ? left : kBK) * ld2);
    }
  }
  // dead_lo / dead_hi (DEAD && kKRow): KDead's bits for the slice
  MJ_DEV u32x4 load(int slice, int i, uint32_t dead_lo = 0, uint32_t dead_hi = 0) const {
    if (LAYOUT == kRowK) {
      const int k0 = slice * kBK;
      return __builtin_amdgcn_raw_buffer_load_b128(rsrc, k0 < klimit ? goff[i] : kOob, k0 * 2, 0);
    }
    uint32_t off = col_ok ? goff[i] : kOob;
    if (DEAD)   // bit 8 (i % 4) of the shifted word set: the offset becomes one that every descriptor rejects
      off |= (uint32_t)__builtin_amdgcn_sbfe((int)(i < 4 ? dead_lo : dead_hi), 8 * (i & 3), 1) & kOob;
    return __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
  }
  MJ_DEV void store(char* stage, int i, u32x4 v) const {
    if (LAYOUT == kRowK)
      *(u32x4*)(stage + st_off + i * RPP * 128) = v;
    else
      *(u32x4*)(stage + ((i & 1) ? st_off1 : st_off) + i * KPP * (ROWS * 2)) = v;
  }
  // one 8-byte half of chunk i (kRowK): an LDS write holds the wavefront's issue while its data
  // leaves the registers (12 cycles per 16-byte write measured between matrix instructions, 5 per 8-byte one)
  MJ_DEV void store_half(char* stage, int i, u32x4 v, int h) const {
    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
    const u32x2 w = {v[2 * h], v[2 * h + 1]};
    if (LAYOUT == kRowK)
      *(u32x2*)(stage + st_off + i * RPP * 128 + h * 8) = w;
    else
      *(u32x2*)(stage + ((i & 1) ? st_off1 : st_off) + i * KPP * (ROWS * 2) + h * 8) = w;
  }
  // MFMA fragment f (32 rows) of k-step ks.
  MJ_DEV bf16x8 frag(const char* stage, int f, int ks) const {
    if (LAYOUT == kRowK) return *(const bf16x8*)(stage + rd[ks] + f * 32 * 128);
    typedef __attribute__((address_space(3))) s16x4* lds_s16x4_ptr;
    const char* p = stage + rd[f] + ks * 16 * (ROWS * 2);
    const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)p);
    const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s16x4_ptr)(p + 4 * (ROWS * 2)));
    const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    return __builtin_bit_cast(bf16x8, v);
  }
};

template <int V>
struct IntTag { static constexpr int value = V; };

// Mask of all-zero k-rows for operands in the kKRow layout (256-row tiles, 256 threads: a thread
// loads chunk i of a slice from k-row t / 32 + 8 i).  One 64-bit word per slice, bit r set = k-row r
// of the slice is zero.  The word of the next slice is requested while the current one is used;
// lo / hi hold the current word shifted so that bit 8 (i % 4) of (i < 4 ? lo : hi) is chunk i's row.
struct KDead {
  __amdgpu_buffer_rsrc_t rsrc;
  uint64_t next;
  uint32_t lo, hi;
  int krow;
  MJ_DEV uint64_t word(int slice) const {
    typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
    const u32x2 w = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(rsrc, 0, slice * 8, 0));
    return ((uint64_t)w[1] << 32) | w[0];
  }
  MJ_DEV void init(const uint64_t* words, int K, int t) {
    krow = t >> 5;
    rsrc = make_rsrc(words, (int64_t)((K + kBK - 1) / kBK) * 8);   // words past K read 0: nothing to skip
    next = word(0);
    lo = hi = 0;
  }
  MJ_DEV void slice_begin(int slice) {
    const uint64_t w = next >> krow;
    lo = (uint32_t)w;
    hi = (uint32_t)(w >> 32);
    next = word(slice + 1);
  }
};

// DEPTH: slices in flight between global memory and the LDS.  1: the loads of slice k+2 are issued
// during slice k and written to the LDS during slice k+1 (one slice of math to land).  2: a second
// set of staging registers; the loads of slice k+3 are issued during slice k and written during
// slice k+2 (two slices to land) -- for shapes whose operands come from HBM on every slice.
template <int BM, int BN, int LAY_A = kRowK, int LAY_B = kRowK, int DEPTH = 1, int WAVES_M = 2, int WAVES_N = 2>
struct GemmTN {
  static_assert(BM % 32 == 0 && BN % 32 == 0, "tile sides are multiples of 32");
  static constexpr int kWavesM = WAVES_M, kWavesN = WAVES_N;
  static constexpr int kThreads = 64 * WAVES_M * WAVES_N;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;   // wavefront tile
  static constexpr int MI = WM / 32, NI = WN / 32;   // 32x32 blocks per wavefront
  using OpA = Operand<BM, LAY_A, kThreads>;
  using OpB = Operand<BN, LAY_B, kThreads>;
  static constexpr int A_LD = OpA::LD, B_LD = OpB::LD;
  static constexpr int LPS = A_LD + B_LD;            // 16-byte chunks per thread per slice
  static constexpr int kStageBytes = OpA::kBytes + OpB::kBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  static_assert(kLdsBytes <= 160 * 1024, "LDS is 160 KB per CU");

  // acc[mi][ni][r]: row = mi*32 + (r/4)*8 + (lane/32)*4 + r%4, col = ni*32 + lane%32
  // within the wavefront tile whose origin is (wm*WM, wn*WN).
  f32x16 acc[MI][NI];

  // A, B: tile origin pointers (row 0 of the tile, k = k_begin); rows_*: valid rows of the tile;
  // ld*: elements between rows (kRowK) or between k-rows (kKRow); K: k extent from the origin.
  // tid: the thread's index in the workgroup (a kernel that loops over tiles passes a value the
  // compiler cannot see through, so that the per-thread address arithmetic is redone per tile
  // instead of living in registers across the epilogue).
  MJ_DEV void run(const __bf16* A, int rows_a, int64_t lda, const __bf16* B, int rows_b,
                  int64_t ldb, int K, char* smem, int tid = threadIdx.x) {
    if (DEPTH == 2) {
      run_deep(A, rows_a, lda, B, rows_b, ldb, K, smem, tid);
      return;
    }
    const int wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    OpA a;
    OpB b;
    a.init(A, rows_a, lda, K, wm * WM, tid);
    b.init(B, rows_b, ldb, K, wn * WN, tid);
    auto slices_begin = [&](int slice) {
      a.slice_begin(slice);
      b.slice_begin(slice);
    };

    u32x4 staged[LPS];
    auto load_one = [&](int slice, int j) {
      if (j < A_LD) staged[j] = a.load(slice, j);
      else staged[j] = b.load(slice, j - A_LD);
    };
    auto store_one = [&](int slice, int j) {
      char* stage = smem + (slice & 1) * kStageBytes;
      if (j < A_LD) a.store(stage, j, staged[j]);
      else b.store(stage + OpA::kBytes, j - A_LD, staged[j]);
    };
    bf16x8 fa[2][MI], fb[2][NI];
    auto read_one = [&](int slice, int ks, int buf, int g) {   // fragment g of the MI + NI
      const char* stage = smem + (slice & 1) * kStageBytes;
      if (g < MI) fa[buf][g] = a.frag(stage, g, ks);
      else fb[buf][g - MI] = b.frag(stage + OpA::kBytes, g - MI, ks);
    };
    // One k-step, hand-scheduled: MI+NI groups, each = [LDS write of one staged chunk of the next
    // slice, then the global load that refills that staging register with the slice after it]
    // + the LDS read of one of the next k-step's fragments + this k-step's share of MFMAs.  The
    // fences keep the groups in this order, so the MFMA pipe always has work queued behind every
    // memory instruction.  `first` is the index of this k-step's first staged chunk (>= LPS: none).
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
    slices_begin(0);
#pragma unroll
    for (int j = 0; j < LPS; ++j) load_one(0, j);
    slices_begin(1);
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
      slices_begin(kt + 2);
      kstep(0, kt, 1, kt, 0);
      kstep(1, kt, 2, kt, G);
      kstep(0, kt, 3, kt, 2 * G);
      wait_lgkmcnt0();                  // own reads of slice kt and writes of slice kt+1 are done
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      kstep(1, kt + 1, 0, kt, LPS);
    }
  }

  // DEPTH == 2 (see the struct's comment).  Iteration kt stores slice kt+1 from staging set
  // (kt+1) & 1 and refills that set with slice kt+3; the loop is unrolled by two so that the set
  // index is a compile-time constant.
  MJ_DEV void run_deep(const __bf16* A, int rows_a, int64_t lda, const __bf16* B, int rows_b, int64_t ldb,
                       int K, char* smem, int tid) {
    const int wave = tid >> 6;
    const int wm = wave % WAVES_M, wn = wave / WAVES_M;
    OpA a;
    OpB b;
    a.init(A, rows_a, lda, K, wm * WM, tid);
    b.init(B, rows_b, ldb, K, wn * WN, tid);
    auto slices_begin = [&](int slice) {
      a.slice_begin(slice);
      b.slice_begin(slice);
    };

    u32x4 staged[2][LPS];
    auto load_one = [&](auto set, int slice, int j) {
      constexpr int S = decltype(set)::value;
      if (j < A_LD) staged[S][j] = a.load(slice, j);
      else staged[S][j] = b.load(slice, j - A_LD);
    };
    auto store_one = [&](auto set, int slice, int j) {
      constexpr int S = decltype(set)::value;
      char* stage = smem + (slice & 1) * kStageBytes;
      if (j < A_LD) a.store(stage, j, staged[S][j]);
      else b.store(stage + OpA::kBytes, j - A_LD, staged[S][j]);
    };
    bf16x8 fa[2][MI], fb[2][NI];
    auto read_one = [&](int slice, int ks, int buf, int g) {
      const char* stage = smem + (slice & 1) * kStageBytes;
      if (g < MI) fa[buf][g] = a.frag(stage, g, ks);
      else fb[buf][g - MI] = b.frag(stage + OpA::kBytes, g - MI, ks);
    };
    constexpr int G = MI + NI, T = MI * NI;
    auto kstep = [&](auto set, int buf, int next_slice, int next_ks, int kt, int first) {
#pragma unroll
      for (int g = 0; g < G; ++g) {
        if (first + g < LPS) {
          store_one(set, kt + 1, first + g);
          load_one(set, kt + 3, first + g);
        }
        read_one(next_slice, next_ks, buf ^ 1, g);
#pragma unroll
        for (int p = g * T / G; p < (g + 1) * T / G; ++p)
          acc[p / NI][p % NI] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[buf][p / NI], fb[buf][p % NI],
                                                                        acc[p / NI][p % NI], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    auto iteration = [&](auto set, int kt) {
      slices_begin(kt + 3);
      kstep(set, 0, kt, 1, kt, 0);
      kstep(set, 1, kt, 2, kt, G);
      kstep(set, 0, kt, 3, kt, 2 * G);
      wait_lgkmcnt0();                  // own reads of slice kt and writes of slice kt+1 are done
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
      kstep(set, 1, kt + 1, 0, kt, LPS);
    };

#pragma unroll
    for (int mi = 0; mi < MI; ++mi)
#pragma unroll
      for (int ni = 0; ni < NI; ++ni)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mi][ni][r] = 0.f;

    const int KT = (K + kBK - 1) / kBK;
    slices_begin(0);
#pragma unroll
    for (int j = 0; j < LPS; ++j) load_one(IntTag<0>(), 0, j);
    slices_begin(1);
#pragma unroll
    for (int j = 0; j < LPS; ++j) load_one(IntTag<1>(), 1, j);
    slices_begin(2);
#pragma unroll
    for (int j = 0; j < LPS; ++j) {
      store_one(IntTag<0>(), 0, j);
      load_one(IntTag<0>(), 2, j);
    }
    wait_lgkmcnt0();
    __builtin_amdgcn_s_barrier();       // slice 0 is in LDS, slices 1 and 2 are on their way to the registers
#pragma unroll
    for (int g = 0; g < G; ++g) read_one(0, 0, 0, g);
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
      iteration(IntTag<1>(), kt);       // even kt: slice kt+1 waits in set 1
      iteration(IntTag<0>(), kt + 1);
    }
    if (kt < KT) iteration(IntTag<1>(), kt);
  }
};

// The same 256 x 256 tile on v_mfma_f32_16x16x32_bf16, in the order that the instruction rewards.
// A wavefront's 128 x 128 is 8 x 8 blocks of 16 x 16 and a 64-wide slice is two k-steps of 32.  The
// two k-steps of a block are issued back to back on the same accumulator: the second instruction
// takes the first one's result inside the matrix unit, so the accumulator is read from and written
// to the register file once per slice instead of once per instruction.  Measured in an MFMA-only
// loop at the socket power limit with random operands: 2146-2188 TFLOP/s in this order against
// 1817-1874 with the accumulators in rotation (which is also held at 82 % of the issue rate by the
// accumulator reads) and 1840 for v_mfma_f32_32x32x16_bf16 in either order.
//
// Blocks are walked row by row (i outer, j inner).  The B fragments of the whole slice stay in
// registers (8 x 2 fragments); the A fragments of row i + 1 are read while row i computes (three
// register pairs in rotation); the last two rows are walked column by column and each B fragment
// pair is re-read for the next slice after its last use.  One barrier per slice, before those two
// rows; the loop body runs from that barrier to the next one (a period, see run()) and carries the LDS
// writes of the next slice and the global loads of the one after it, one slice in flight between
// global memory and the LDS (a ring of 24 staging registers with one and a half slices in flight
// measured 7 % slower: more requests in flight only lengthen each one).
//
// The matrix instructions are written as assembly so that the result register IS the accumulator
// operand: with all 256 accumulation registers taken the register allocator otherwise routes some
// blocks through copies (and the wait states those need).  The first slice starts from the constant
// 0, so nothing but these instructions ever writes an accumulator.  The compiler does not see matrix
// instructions inside the assembly, so the wait states it would put between one of them and an
// ordinary instruction that touches an accumulator (7 behind a four-pass instruction, 2 in front)
// are spelled out where such an instruction can follow or precede: behind the last block of a period
// and of the last two rows (loop exit; copies on the back edge, should the allocator ever make any)
// and in front of a period's first block.  They cost nothing: a block keeps the matrix unit busy for
// 32 cycles.
template <int BM, int BN, int LAY_A = kRowK, int LAY_B = kRowK, bool DEAD_A = false, bool DEAD_B = false>
struct GemmTN16 {
  static_assert(BM == 256 && BN == 256, "four wavefronts of 128 x 128");
  static constexpr int kThreads = 256;
  static constexpr int WM = 128, WN = 128;
  static constexpr int MI = 8, NI = 8;               // 16 x 16 blocks per wavefront
  using OpA = Operand<BM, LAY_A, kThreads, DEAD_A, 16>;
  using OpB = Operand<BN, LAY_B, kThreads, DEAD_B, 16>;
  static constexpr int A_LD = OpA::LD, B_LD = OpB::LD, LPS = A_LD + B_LD;
  static constexpr int kStageBytes = OpA::kBytes + OpB::kBytes;
  static constexpr int kLdsBytes = 2 * kStageBytes;
  // a mask over k-rows comes with a k-major A; it is read once and would serve a k-major B as well
  static constexpr bool kKDead = DEAD_A && LAY_A == kKRow;
  static_assert(!(DEAD_B && LAY_B == kKRow), "k-row masks are handed in with A");
  static_assert(LPS <= 16, "three memory instructions per staged chunk in the 48 blocks of the first period");

  // acc[mi][ni][r]: row = mi*16 + (lane/16)*4 + r, col = ni*16 + lane%16 within the wavefront tile
  f32x4 acc[MI][NI];

  // register pair of the A fragments of row i: rows 6 and 7 are in use together, and row 0 of the
  // next slice is read while they are
  static constexpr int slot(int i) { return i == 0 ? 2 : i == 5 ? 2 : (i & 1) ? 0 : 1; }

  MJ_DEV void run(const __bf16* A, int rows_a, int64_t lda, const __bf16* B, int rows_b, int64_t ldb, int K,
                  char* smem, int tid = threadIdx.x, const uint64_t* dead_a = nullptr,
                  const uint64_t* dead_b = nullptr) {
    const int wave = tid >> 6;
    const int wm = wave & 1, wn = wave >> 1;
    OpA a;
    OpB b;
    a.init(A, rows_a, lda, K, wm * WM, tid, dead_a);
    b.init(B, rows_b, ldb, K, wn * WN, tid, dead_b);
    a.init16(wm * WM, tid);
    b.init16(wn * WN, tid);
    KDead kd;
    if (kKDead) kd.init(dead_a, K, tid);
    auto slices_begin = [&](int slice) {     // in slice order: the mask word of the next slice is requested here
      a.slice_begin(slice);
      b.slice_begin(slice);
      if (kKDead) kd.slice_begin(slice);
    };

    u32x4 staged[LPS];
    auto load_one = [&](int slice, int j) {
      if (j < A_LD) staged[j] = kKDead ? a.load(slice, j, kd.lo, kd.hi) : a.load(slice, j);
      else staged[j] = b.load(slice, j - A_LD);
    };
    auto store_one = [&](int slice, int j) {
      char* stage = smem + (slice & 1) * kStageBytes;
      if (j < A_LD) a.store(stage, j, staged[j]);
      else b.store(stage + OpA::kBytes, j - A_LD, staged[j]);
    };
    auto store_half = [&](int slice, int j, int h) {
      char* stage = smem + (slice & 1) * kStageBytes;
      if (j < A_LD) a.store_half(stage, j, staged[j], h);
      else b.store_half(stage + OpA::kBytes, j - A_LD, staged[j], h);
    };
    bf16x8 fa[3][2], fb[NI][2];
    auto read_a_half = [&](int slice, int i, int ks) {
      const char* stage = smem + (slice & 1) * kStageBytes;
      fa[slot(i)][ks] = a.frag16(stage, i, ks);
    };
    auto read_b = [&](int slice, int j) {
      const char* stage = smem + (slice & 1) * kStageBytes + OpA::kBytes;
      fb[j][0] = b.frag16(stage, j, 0);
      fb[j][1] = b.frag16(stage, j, 1);
    };
    // first: the k-step 0..31 of block (i, j); second: its k-step 32..63, on the first one's result.
    // The second cannot issue before the first has gone through the matrix unit (16 cycles): a block's
    // memory instruction sits between the two, where the wavefront would otherwise wait.
    auto first = [&](auto init, auto lead, int i, int j) {
      constexpr bool kInit = decltype(init)::value != 0, kLead = decltype(lead)::value != 0;
      (void)fa; (void)fb; (void)acc;     // named outside the assembly too, so that the lambda captures them
      if constexpr (kInit)
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, 0" : "=a"(acc[i][j]) : "v"(fa[slot(i)][0]), "v"(fb[j][0]));
      else if constexpr (kLead)
        asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fa[slot(i)][0]), "v"(fb[j][0]));
      else
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fa[slot(i)][0]), "v"(fb[j][0]));
    };
    auto second = [&](auto settle, int i, int j) {
      constexpr bool kSettle = decltype(settle)::value != 0;
      (void)fa; (void)fb; (void)acc;
      if constexpr (kSettle)
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0\n\ts_nop 9" : "+a"(acc[i][j]) : "v"(fa[slot(i)][1]), "v"(fb[j][1]));
      else
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[i][j]) : "v"(fa[slot(i)][1]), "v"(fb[j][1]));
    };

    const int KT = (K + kBK - 1) / kBK;
    slices_begin(0);
#pragma unroll
    for (int j = 0; j < LPS; ++j) load_one(0, j);
    slices_begin(1);
#pragma unroll
    for (int j = 0; j < LPS; ++j) {
      store_one(0, j);
      load_one(1, j);
    }
    wait_lgkmcnt0();
    __builtin_amdgcn_s_barrier();       // slice 0 is in LDS, slice 1 is on its way to the registers
    read_a_half(0, 0, 0);
    read_a_half(0, 0, 1);
#pragma unroll
    for (int j = 0; j < NI; ++j) read_b(0, j);

    // A period runs from the barrier inside slice s-1 to the one inside slice s: rows 6, 7 of slice
    // s-1, then rows 0..5 of slice s: 64 blocks.  During it slice s+1 moves from the staging registers
    // to the LDS stage that slice s-1 has just left, and slice s+2 is loaded: per 16-byte chunk two
    // 8-byte LDS writes and one global load, each in the gap INSIDE a block (between its two matrix
    // instructions, where 12 issue cycles are free anyway), three blocks out of four.  The first
    // period has no rows 6, 7: its 48 blocks carry one memory instruction each.
    auto mem_op = [&](int s, int slot, bool first_period) {
      const int q = first_period ? slot - 16 : slot;              // 0..47 or 0..63
      const int c = first_period ? q / 3 : q / 4, r = first_period ? q % 3 : q % 4;
      if (q < 0 || c >= LPS) return;
      if (r == 0) store_half(s + 1, c, 0);
      if (r == 1) store_half(s + 1, c, 1);
      if (r == 2) load_one(s + 2, c);
    };
    // One block: its two matrix instructions with the period's memory instruction `slot` between them.
    auto block = [&](auto init, auto lead, auto settle, int i, int j, int s, int slot, bool first_period) {
      first(init, lead, i, j);
      __builtin_amdgcn_sched_barrier(0);
      mem_op(s, slot, first_period);
      __builtin_amdgcn_sched_barrier(0);
      second(settle, i, j);
      __builtin_amdgcn_sched_barrier(0);
    };
    // Rows 6 and 7 of slice s-1, column by column, so that the B pairs are released one per two blocks:
    // each is re-read for slice s after its last use (behind the next column's first block; the last
    // one inside row 0).  more: slice s exists (its fragments are read, the period's memory
    // instructions ride along).
    auto rows_back = [&](auto init, auto more, int s) {
      constexpr bool kMore = decltype(more)::value != 0;
      if (kMore) slices_begin(s + 2);   // the period's loads
#pragma unroll
      for (int j = 0; j < NI; ++j) {
        if (j == 0) block(init, IntTag<1>(), IntTag<0>(), MI - 2, j, s, kMore ? 2 * j : -1, false);
        else block(init, IntTag<0>(), IntTag<0>(), MI - 2, j, s, kMore ? 2 * j : -1, false);
        if (kMore) {
          if (j < 2) read_a_half(s, 0, j);
          if (j > 0) read_b(s, j - 1);
          __builtin_amdgcn_sched_barrier(0);
        }
        if (j == NI - 1) block(init, IntTag<0>(), IntTag<1>(), MI - 1, j, s, kMore ? 2 * j + 1 : -1, false);
        else block(init, IntTag<0>(), IntTag<0>(), MI - 1, j, s, kMore ? 2 * j + 1 : -1, false);
      }
    };
    // Rows 0..5 of slice s; the A pair of row i+1 is read meanwhile (row 5: of rows 6 and 7).
    auto rows_front = [&](auto init, int s, bool first_period) {
      if (first_period) slices_begin(s + 2);
#pragma unroll
      for (int i = 0; i < MI - 2; ++i)
#pragma unroll
        for (int j = 0; j < NI; ++j) {
          if (i == MI - 3 && j == NI - 1) block(init, IntTag<0>(), IntTag<1>(), i, j, s, 16 + i * NI + j, first_period);
          else block(init, IntTag<0>(), IntTag<0>(), i, j, s, 16 + i * NI + j, first_period);
          if (j < 2) read_a_half(s, i + 1, j);
          if (i == 5 && (j == 2 || j == 3)) read_a_half(s, 7, j - 2);
          if (i == 0 && j == 2 && !first_period) read_b(s, NI - 1);   // the last B pair, left over by rows_back
          __builtin_amdgcn_sched_barrier(0);
        }
    };
    auto publish = [&]() {
      wait_lgkmcnt0();                  // own reads of the slice that ends and writes of the next one are done
      __builtin_amdgcn_s_barrier();
      __builtin_amdgcn_sched_barrier(0);
    };
    // Every accumulator is first written at exactly one place (rows 0..5: the first period; rows 6, 7:
    // the second one, which with a single slice reads the zero-filled stage of a slice past K and
    // starts loads that the buffer descriptors reject).
    rows_front(IntTag<1>(), 0, true);
    publish();
    rows_back(IntTag<1>(), IntTag<1>(), 1);
    if (KT > 1) {
      rows_front(IntTag<0>(), 1, false);
      for (int s = 2; s < KT; ++s) {
        publish();
        rows_back(IntTag<0>(), IntTag<1>(), s);
        rows_front(IntTag<0>(), s, false);
      }
      rows_back(IntTag<0>(), IntTag<0>(), KT);
    }
  }
};

}  // namespace mj
