// Pieces shared by the two prefill GEMM kernels: the workgroup -> tile map (tile_map.h)
// and the per-wave epilogue.
#pragma once
#include "device_utils.h"
#include "tile_map.h"

namespace tlhip {

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
