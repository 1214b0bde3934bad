// Pieces shared by the two prefill GEMM kernels: the workgroup -> tile map and
// the per-wave epilogue.
#pragma once
#include <algorithm>

#include "device_utils.h"

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
__device__ __forceinline__ bool tile_of(const TileMap& t, int id, int& tm, int& tn) {
  const int s_shift = t.gm_shift + t.gn_shift;
  const int xcd = id & 7, local = id >> 3;
  const int sb = (local >> s_shift) * 8 + xcd;
  const int in = local & ((1 << s_shift) - 1);
  const int sb_n = sb / t.sbm, sb_m = sb - sb_n * t.sbm;
  tm = (sb_m << t.gm_shift) + (in & ((1 << t.gm_shift) - 1));
  tn = (sb_n << t.gn_shift) + (in >> t.gm_shift);
  return sb < t.nsb && tm < t.tiles_m && tn < t.tiles_n;
}

struct OutArgs {
  void* y;
  int y_dtype;
  int vec_ok;  // N % 8 == 0 and y 16-byte aligned: rows can be stored 8 columns at a time
  int m, n;
  float alpha;
  DevEpilogue epi;
  const float* col_scale;  // null, or one f32 factor per output column, applied with alpha (int8-row: the row scales of W)
};

// Defined in gemm_direct.hip: the second launch of a K-sliced tiled GEMM.
int launch_k_slice_reduce(int ks, const float* planes, const OutArgs& o, hipStream_t stream);

// Epilogue of one 32-row block of a wave: TN accumulator tiles of
// v_mfma_f32_32x32x16 side by side (32 x 32*TN outputs).  The accumulator layout
// (lane l: column l%32, rows 8*(r/4) + 4*(l/32) + r%4) would give 64-byte row
// pieces per store; instead the block goes through a private LDS patch and every
// lane then owns 8 consecutive columns of one row: acc*alpha -> ops in order
// (bias indexed by n, unary) -> cast, stored as one 16-byte (f16) or two 16-byte
// (f32) pieces, whole 128-byte lines per row for f16 and TN = 2.
// `patch` holds 32 * (32*TN + 4) floats and belongs to this wave alone.
// `plane` != null (a K slice of a K-sliced launch): the bare sums go to that M x N f32
// plane instead, no alpha, no ops; `o` then only gives the shape.  (A modified copy of
// `o` would do the same, but a copy of the kernel arguments whose op arrays are indexed
// at run time lands in scratch memory.)
// PLANE = false: instances that never take K slices compile without the choice.
// COLSCALE: o.col_scale holds a factor per column (never null then); a K slice leaves it,
// like alpha, to the launch that adds the planes.
template <int TN, bool PLANE = false, bool COLSCALE = false>
__device__ __forceinline__ void wave_epilogue(float* patch, const float16_t (&acc)[TN], int lane, int row0,
                                              int col0, const OutArgs& o, float* plane = nullptr) {
  const bool bare = PLANE && plane != nullptr;  // uniform
  // read where they are used (with PLANE = false exactly the kernel-argument reads of before:
  // hoisted copies cost scalar registers, and the largest instances have none to spare)
  auto out_base = [&]() -> void* { return bare ? (void*)plane : o.y; };
  auto out_dtype = [&]() -> int { return bare ? (int)TLHIP_F32 : o.y_dtype; };
  auto out_alpha = [&]() -> float { return bare ? 1.f : o.alpha; };
  constexpr int PW = TN * 32 + 4;
  constexpr int LPR = TN * 4;     // lanes per row, 8 columns each
  constexpr int RPP = 64 / LPR;   // rows per pass (TN = 3: 5 rows on 60 lanes, four lanes idle)
  constexpr int PASSES = (32 + RPP - 1) / RPP;
  const int lrow = lane & 31, lk = lane >> 5;
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) patch[(8 * (r >> 2) + 4 * lk + (r & 3)) * PW + j * 32 + lrow] = acc[j][r];
  __builtin_amdgcn_s_waitcnt(0xc07f);  // this wave's LDS writes have landed (lgkmcnt(0))
  const int rr0 = lane / LPR, cc = (lane % LPR) * 8;
  const bool lane_used = rr0 < RPP;
  const int col = col0 + cc;
  const bool vec = (bare ? o.n % 8 == 0 : o.vec_ok != 0) && col + 8 <= o.n;
  // The common chain, [bias] then [unary], keeps the lane's 8 bias values in
  // registers across the passes (the column does not change) and runs no loop
  // over the ops per element.
  const int n_ops = bare ? 0 : o.epi.n_ops;
  const bool has_bias = n_ops >= 1 && o.epi.kind[0] == TLHIP_EPI_BIAS;
  const int un_at = has_bias ? 1 : 0;
  const bool simple = n_ops <= un_at + 1 && (n_ops == un_at || o.epi.kind[un_at] == TLHIP_EPI_UNARY);
  const int unary = (simple && n_ops > un_at) ? o.epi.unary[un_at] : TLHIP_UNARY_NONE;
  float cscale[COLSCALE ? 8 : 1];  // alpha x the lane's column factors
  if constexpr (COLSCALE) {
#pragma unroll
    for (int e = 0; e < 8; ++e) cscale[e] = bare ? 1.f : o.alpha * o.col_scale[min(col + e, o.n - 1)];
  }
  auto scale_of = [&](int e) -> float {
    if constexpr (COLSCALE) return cscale[e];
    else return out_alpha();
  };
  float bias[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    bias[e] = 0.f;
    if (simple && has_bias && col + e < o.n) {
      if (o.epi.input_dtype[0] == TLHIP_F16) bias[e] = (float)((const _Float16*)o.epi.input[0])[col + e];
      else bias[e] = ((const float*)o.epi.input[0])[col + e];
    }
  }
#pragma unroll 1
  for (int p = 0; p < PASSES; ++p) {
    const int rr = min(p * RPP + rr0, 31);
    const int row = row0 + rr;
    const float4_t a = *(const float4_t*)(patch + rr * PW + cc);
    const float4_t b = *(const float4_t*)(patch + rr * PW + cc + 4);
    float v[8] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
    if (row < o.m && lane_used && p * RPP + rr0 < 32) {
      if (simple) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = apply_unary(unary, v[e] * scale_of(e) + bias[e]);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c = min(col + e, o.n - 1);
          v[e] = apply_epilogue(o.epi, v[e] * scale_of(e), c, (int64_t)row * o.n + c);
        }
      }
      if (vec) {
        const int64_t idx = (int64_t)row * o.n + col;
        if (out_dtype() == TLHIP_F16) {
          half8_t h;
#pragma unroll
          for (int e = 0; e < 8; ++e) h[e] = (_Float16)v[e];
          __builtin_nontemporal_store(h, (half8_t*)((_Float16*)out_base() + idx));  // written once, not read back: 0.5-1.5 % faster
        } else {
          float* dst = (float*)out_base() + idx;
          __builtin_nontemporal_store((float4_t){v[0], v[1], v[2], v[3]}, (float4_t*)dst);
          __builtin_nontemporal_store((float4_t){v[4], v[5], v[6], v[7]}, (float4_t*)(dst + 4));
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (col + e < o.n) store_out(out_base(), out_dtype(), (int64_t)row * o.n + col + e, v[e]);
      }
    }
  }
  __builtin_amdgcn_s_waitcnt(0xc07f);  // reads done before the patch is overwritten
}

}  // namespace tlhip
