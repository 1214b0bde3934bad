// Pieces shared by the two matrix-core GEMV kernels (gemv_mfma.hip,
// gemv_mfma_xreg.hip).
#pragma once
#include "device_utils.h"

namespace tlhip {
namespace {

__device__ __forceinline__ half8_t join8(const half2_t (&h)[4]) {
  half8_t r;
  r[0] = h[0][0]; r[1] = h[0][1]; r[2] = h[1][0]; r[3] = h[1][1];
  r[4] = h[2][0]; r[5] = h[2][1]; r[6] = h[3][0]; r[7] = h[3][1];
  return r;
}

// 4x4 transpose of 32-bit words across the four lanes l, l+16, l+32, l+48:
// afterwards register i of lane-group g holds what register g of lane-group i
// held.  Two swap stages: distance 32 on register pairs (0,2) (1,3), then
// distance 16 on pairs (0,1) (2,3).
__device__ __forceinline__ void transpose4(uint32_t& r0, uint32_t& r1, uint32_t& r2, uint32_t& r3) {
  // v_permlane32_swap: lanes 32..63 of the first operand <-> lanes 0..31 of the second
  auto s02 = __builtin_amdgcn_permlane32_swap(r0, r2, false, false);
  r0 = s02[0]; r2 = s02[1];
  auto s13 = __builtin_amdgcn_permlane32_swap(r1, r3, false, false);
  r1 = s13[0]; r3 = s13[1];
  // v_permlane16_swap: odd 16-lane rows of the first operand <-> even rows of the second
  auto s01 = __builtin_amdgcn_permlane16_swap(r0, r1, false, false);
  r0 = s01[0]; r1 = s01[1];
  auto s23 = __builtin_amdgcn_permlane16_swap(r2, r3, false, false);
  r2 = s23[0]; r3 = s23[1];
}

// The last arriver's sum over the ks (a power of two >= 2) published tiles of a row
// block, in slice order.  `tiles` + sl*stride + at + 16*q (q = 0..3) are this lane's four
// values of slice sl.  The loads of four slices are issued together: one load per
// loop iteration (the sum needs it at once) made every slice a round trip to L2 of
// its own, about 1 us each.
__device__ __forceinline__ float4_t sum_slices(const float* tiles, int ks, int at, int stride = 256) {
  float4_t sum = {0.f, 0.f, 0.f, 0.f};
  for (int sl0 = 0; sl0 < ks; sl0 += 4) {
    float v[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int sl = min(sl0 + j, ks - 1);  // ks = 2: the second slice again, not added below
#pragma unroll
      for (int q = 0; q < 4; ++q)
        v[j][q] = __hip_atomic_load(tiles + sl * stride + at + 16 * q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const bool keep = sl0 + j < ks;
#pragma unroll
      for (int q = 0; q < 4; ++q) sum[q] += keep ? v[j][q] : 0.f;
    }
  }
  return sum;
}

}  // namespace
}  // namespace tlhip
