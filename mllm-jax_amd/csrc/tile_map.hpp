// tile_map.hpp -- work-item id -> (tile row, tile column, k-split) of the tile kernels.
//
// Plain C++ (no HIP header): the kernels include it through gemm_tn.hpp, and a host-only build
// under the address / undefined-behaviour sanitizers walks every id of a sweep of problems.
#pragma once

#if defined(__HIPCC__)
#define MJ_HD __host__ __device__ inline
#else
#define MJ_HD inline
#endif

namespace mj {

// Maps a linear work-item id to a tile (and a k-split) so that (a) the 32 items that the
// workgroups of one XCD work on at the same time (ids congruent mod 8 go to the same XCD) form a
// 2^lgm x 2^lgn x 2^lgs block of (tile rows, tile columns, k-splits), lgm + lgn + lgs = 5, whose
// tiles share operand slices in that XCD's L2, and (b) consecutive blocks -- the ones the eight
// XCDs work on at the same time -- walk along N first (n_first) or along M first.  The blocks of
// all k-splits form one list.  Slots of a block that fall outside the problem are ids whose
// workgroups leave at once; pick_shape() chooses the block shape with the fewest of them (they cost
// a workgroup launch each, which is what small problems are made of), preferring 4 x 8 x 1, the
// shape with the fewest operand panels per tile.
struct TileMap {
  int tiles_m, tiles_n, sb_m, sb_n, n_first, lgm, lgn, lgs, splits;
  MJ_HD TileMap(int tm, int tn, int n_first_ = 0, int lgm_ = 2, int splits_ = 1, int lgs_ = 0)
      : tiles_m(tm), tiles_n(tn), sb_m((tm + (1 << lgm_) - 1) >> lgm_),
        sb_n((tn + (1 << (5 - lgm_ - lgs_)) - 1) >> (5 - lgm_ - lgs_)), n_first(n_first_), lgm(lgm_),
        lgn(5 - lgm_ - lgs_), lgs(lgs_), splits(splits_) {}
  MJ_HD int split_blocks() const { return (splits + (1 << lgs) - 1) >> lgs; }
  MJ_HD int blocks() const { return sb_m * sb_n * split_blocks(); }
  MJ_HD int items() const { return (blocks() + 7) / 8 * 8 * 32; }
  MJ_HD bool tile(int pid, int& tm, int& tn, int& split) const {
    const int xcd = pid & 7, q = pid >> 3;
    const int sbg = (q >> 5) * 8 + xcd, within = q & 31, per = sb_m * sb_n;
    if (sbg >= per * split_blocks()) return false;
    const int sblk = sbg / per;
    const int sb = sbg - sblk * per;
    const int bm = n_first ? sb / sb_n : sb % sb_m, bn = n_first ? sb % sb_n : sb / sb_m;
    tm = (bm << lgm) + (within & ((1 << lgm) - 1));
    tn = (bn << lgn) + ((within >> lgm) & ((1 << lgn) - 1));
    split = (sblk << lgs) + (within >> (lgm + lgn));
    return tm < tiles_m && tn < tiles_n && split < splits;
  }
  // Block shape with the fewest slots for tm x tn tiles in `splits` k-splits.
  static TileMap pick_shape(int tm, int tn, int n_first, int splits) {
    int best_m = 2, best_s = 0;
    long best = -1;
    for (int pref = 0; pref < 2; ++pref)            // first pass: the preferred 4 x 8 x 1 only
      for (int ls = 0; ls <= 5; ++ls)
        for (int lm = 0; lm + ls <= 5; ++lm) {
          if (pref == 0 && !(ls == 0 && lm == 2)) continue;
          const TileMap t(tm, tn, n_first, lm, splits, ls);
          const long slots = (long)t.blocks() * 32;
          // a different shape must halve the slots to displace the choice so far: measured, a
          // 16 x 2 block costs a large product 3-6 % (more operand panels per tile) while its empty
          // slots cost nothing, and a 2 x 4 x 4 block makes a 2 x 4-tile, 32-split product 40 % faster
          if (best < 0 || slots * 2 <= best) { best = slots; best_m = lm; best_s = ls; }
        }
    return TileMap(tm, tn, n_first, best_m, splits, best_s);
  }
};

}  // namespace mj
