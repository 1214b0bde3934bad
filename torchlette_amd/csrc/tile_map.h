// The workgroup -> tile map of the prefill GEMMs: host code that shapes it, and the
// function a workgroup calls to find its tile.  No HIP types: a plain C++ compiler can
// include this file (the CPU tests check the map that way).
#pragma once
#include <algorithm>
#include <cstdint>

#ifdef __HIPCC__
#define TLHIP_TILE_MAP_FN __host__ __device__ __forceinline__
#else
#define TLHIP_TILE_MAP_FN inline
#endif

namespace tlhip {

// Workgroup ids are dealt round-robin to the 8 XCDs (each with its own L2), and
// the workgroups of one XCD start in id order.  A run of 2^sb_shift (at most 32 =
// the CUs of an XCD) consecutive workgroups of an XCD takes one "super-block" of
// 2^gm_shift x 2^gn_shift tiles, so the tiles that run together on an XCD share
// their X row blocks and W column blocks through that XCD's L2: the L2 fill per
// K step is GM row blocks of X and GN column blocks of W instead of 32 and 1.
struct TileMap {
  int tiles_m, tiles_n;
  int gm_shift, gn_shift;  // super-block = 2^gm_shift x 2^gn_shift tiles
  int sbm;                 // super-blocks along M
  int nsb;                 // super-blocks in all
};

// Bytes per k that one more row of tiles (an X row block) and one more column of tiles (a
// W column block) add to what an XCD's L2 has to fetch for a super-block.
struct TileCost {
  int x_bytes;  // tile M x 2 (f16 activations)
  int w_bytes;  // tile N x bytes per packed weight
};

// The map with super-blocks of 2^s_shift tiles, of the shape (rows of tiles up to 8, a power
// of two) that fetches the fewest bytes per k for the tiles it really holds; ties go to the
// taller block.  4 x 8 tiles for the large problems of every format; a matrix of few column
// tiles gets blocks as wide as it is (1024 columns on 256 x 128 tiles at M = 6000: 8 x 1
// blocks read X once per column tile, 180 us; 2 x 4 blocks 127 us).
inline TileMap tile_map_with(int tiles_m, int tiles_n, int s_shift, TileCost cost) {
  TileMap t;
  t.tiles_m = tiles_m;
  t.tiles_n = tiles_n;
  int gm_shift = 0;
  int64_t best = -1;
  for (int g = 0; g <= 3 && g <= s_shift; ++g) {
    const int64_t rows = std::min<int64_t>(1 << g, tiles_m), cols = std::min<int64_t>(1 << (s_shift - g), tiles_n);
    const int64_t bytes = rows * cost.x_bytes + cols * cost.w_bytes;
    // per tile really held: a block clipped by the matrix must not look cheap
    const int64_t per_tile = bytes * 1024 / (rows * cols);
    if (best < 0 || per_tile <= best) {
      best = per_tile;
      gm_shift = g;
    }
  }
  t.gm_shift = gm_shift;
  t.gn_shift = s_shift - gm_shift;
  const int gm = 1 << t.gm_shift, gn = 1 << t.gn_shift;
  t.sbm = (tiles_m + gm - 1) / gm;
  const int sbn = (tiles_n + gn - 1) / gn;
  t.nsb = t.sbm * sbn;
  return t;
}

// Tiles of the busiest XCD under a map (super-block sb goes to XCD sb % 8; the ones on the
// edges hold fewer tiles than 2^s_shift).
inline int64_t busiest_xcd_tiles(const TileMap& t) {
  int64_t load[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  const int gm = 1 << t.gm_shift, gn = 1 << t.gn_shift;
  for (int sb = 0; sb < t.nsb; ++sb) {
    const int sb_n = sb / t.sbm, sb_m = sb - sb_n * t.sbm;
    const int rows = t.tiles_m - sb_m * gm < gm ? t.tiles_m - sb_m * gm : gm;
    const int cols = t.tiles_n - sb_n * gn < gn ? t.tiles_n - sb_n * gn : gn;
    load[sb & 7] += (int64_t)rows * cols;
  }
  int64_t most = 0;
  for (int64_t l : load) most = l > most ? l : most;
  return most;
}

// Super-blocks as large as 32 tiles, but at least 16 of them so that every XCD gets work,
// and no larger than keeps the XCDs level: partial super-blocks on the edges can all fall
// to the same XCDs (12 x 20 tiles in super-blocks of 8 x 1: the even XCDs got 40 tiles
// each, the odd ones 20, and a launch that fits the chip in one round took two), so the
// super-blocks shrink until the busiest XCD needs no more rounds of its 32 CUs than the
// whole launch needs of the chip, or, in a launch of more than two rounds, holds at most
// 5 % more than its share.
inline TileMap make_tile_map(int tiles_m, int tiles_n, TileCost cost, int* grid) {
  static thread_local struct {
    int tiles_m = 0, tiles_n = 0, x_bytes = 0, w_bytes = 0, s_shift = 0;
  } last;  // the loop below costs a few microseconds for thousands of tiles
  const int64_t total = (int64_t)tiles_m * tiles_n;
  int s_shift = 5;
  if (last.tiles_m == tiles_m && last.tiles_n == tiles_n && last.x_bytes == cost.x_bytes && last.w_bytes == cost.w_bytes) {
    s_shift = last.s_shift;
  } else {
    while (s_shift > 0 && (total >> s_shift) < 16) --s_shift;
    const int64_t chip_rounds = (total + 255) / 256;
    int best_shift = s_shift;
    int64_t best_load = -1;
    for (int s = s_shift; s >= 0; --s) {
      const int64_t load = busiest_xcd_tiles(tile_map_with(tiles_m, tiles_n, s, cost));
      if (best_load < 0 || load < best_load) {
        best_load = load;
        best_shift = s;
      }
      if ((load + 31) / 32 <= chip_rounds || (chip_rounds > 2 && load * 8 * 20 <= total * 21)) break;
    }
    s_shift = best_shift;
    last.tiles_m = tiles_m;
    last.tiles_n = tiles_n;
    last.x_bytes = cost.x_bytes;
    last.w_bytes = cost.w_bytes;
    last.s_shift = s_shift;
  }
  const TileMap t = tile_map_with(tiles_m, tiles_n, s_shift, cost);
  *grid = ((t.nsb + 7) / 8) * 8 << s_shift;
  return t;
}

// false: this workgroup has no tile (padding of the last super-blocks).
TLHIP_TILE_MAP_FN bool tile_of(const TileMap& t, int id, int& tm, int& tn) {
  const int s_shift = t.gm_shift + t.gn_shift;
  const int xcd = id & 7, local = id >> 3;
  const int sb = (local >> s_shift) * 8 + xcd;
  const int in = local & ((1 << s_shift) - 1);
  const int sb_n = sb / t.sbm, sb_m = sb - sb_n * t.sbm;
  tm = (sb_m << t.gm_shift) + (in & ((1 << t.gm_shift) - 1));
  tn = (sb_n << t.gn_shift) + (in >> t.gm_shift);
  return sb < t.nsb && tm < t.tiles_m && tn < t.tiles_n;
}

}  // namespace tlhip
