// The small ops that sit either side of the packed matmul when the frontend
// calls them unfused (api.linear issues matmul, then add —
// src/frontend/torchlette.ts:887-894 — and the model issues the activation):
// bias add over the last dimension, a unary activation, an f32<->f16 cast, and
// the two producers of a decode Linear's input: RMSNorm
// (src/backend/webgpu/rmsnorm-kernel.ts:31-66) and the MLP's act(gate) * up
// (packages/qwen3-browser/src/model.ts:357-361).  All are one pass over the data.
#include <algorithm>

#include "device_utils.h"

namespace tlhip {
namespace {

template <typename T>
__global__ __launch_bounds__(256) void bias_add_kernel(const T* __restrict__ in, const void* __restrict__ bias,
                                                      int bias_dtype, T* __restrict__ out, int64_t count,
                                                      int64_t n) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < count; i += stride) {
    const int64_t col = i % n;
    const float b = bias_dtype == TLHIP_F16 ? (float)((const _Float16*)bias)[col] : ((const float*)bias)[col];
    out[i] = (T)((float)in[i] + b);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void unary_kernel(int op, const T* __restrict__ in, T* __restrict__ out,
                                                   int64_t count) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < count; i += stride) out[i] = (T)apply_unary(op, (float)in[i]);
}

template <typename S, typename D>
__global__ __launch_bounds__(256) void cast_kernel(const S* __restrict__ in, D* __restrict__ out, int64_t count) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < count; i += stride) out[i] = (D)in[i];
}

template <typename T>
__global__ __launch_bounds__(256) void gated_mul_kernel(int op, const T* __restrict__ gate, const T* __restrict__ up,
                                                       T* __restrict__ out, int64_t count) {
  int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; i < count; i += stride) out[i] = (T)(apply_unary(op, (float)gate[i]) * (float)up[i]);
}

// One workgroup per row.  The row is read twice (the second time from cache):
// once for the sum of squares, once to scale.  f32 arithmetic throughout.
template <typename XT, typename YT>
__global__ __launch_bounds__(256) void rmsnorm_kernel(const XT* __restrict__ x, const float* __restrict__ weight,
                                                     YT* __restrict__ y, int64_t d, float eps) {
  __shared__ float red[4];
  const XT* xr = x + (int64_t)blockIdx.x * d;
  YT* yr = y + (int64_t)blockIdx.x * d;
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < d; i += 256) {
    const float v = (float)xr[i];
    ss = fmaf(v, v, ss);
  }
  ss = group_sum(ss, 64);
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
  __syncthreads();
  const float total = (red[0] + red[1]) + (red[2] + red[3]);
  const float inv = 1.f / sqrtf(total / (float)d + eps);
  for (int64_t i = threadIdx.x; i < d; i += 256) yr[i] = (YT)(((float)xr[i] * inv) * weight[i]);
}

// The rest of an epilogue chain over a finished [M,N] output, in place: a lane takes 8
// consecutive columns of a row (N is a multiple of 8), the output and the steps' inputs in
// 16-byte pieces.
template <typename T>
__global__ __launch_bounds__(256) void epilogue_tail_kernel(T* __restrict__ y, int64_t groups, int64_t n, const DevEpilogue ep) {
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; t < groups; t += stride) {
    const int64_t idx = t * 8;
    const int64_t col = idx % n;
    float v[8];
    if constexpr (sizeof(T) == 2) {
      const half8_t h = *(const half8_t*)(y + idx);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] = (float)h[e];
    } else {
      const float4_t lo = *(const float4_t*)(y + idx), hi = *(const float4_t*)(y + idx + 4);
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = lo[e];
        v[4 + e] = hi[e];
      }
    }
    apply_epilogue_row8(ep, v, col, idx, true, n - 1);
    if constexpr (sizeof(T) == 2) {
      half8_t h;
#pragma unroll
      for (int e = 0; e < 8; ++e) h[e] = (_Float16)v[e];
      *(half8_t*)(y + idx) = h;
    } else {
      *(float4_t*)(y + idx) = (float4_t){v[0], v[1], v[2], v[3]};
      *(float4_t*)(y + idx + 4) = (float4_t){v[4], v[5], v[6], v[7]};
    }
  }
}

int grid_for(int64_t count) {
  const int64_t blocks = (count + 255) / 256;
  const int64_t cap = (int64_t)device_cu_count() * 16;
  return (int)std::max<int64_t>(1, std::min(blocks, cap));
}

}  // namespace

bool epilogue_tail_applicable(const void* y, int64_t n) { return n > 0 && n % 8 == 0 && ((uintptr_t)y & 15) == 0; }

int launch_epilogue_tail(void* y, int y_dtype, int64_t m, int64_t n, const DevEpilogue& ep, hipStream_t stream) {
  if (!epilogue_tail_applicable(y, n)) return set_error(TLHIP_ERR_INVALID, "epilogue tail: N must be a multiple of 8 and the output 16-byte aligned");
  const int64_t groups = m * n / 8;
  if (groups == 0 || ep.n_ops == 0) return TLHIP_OK;
  const int grid = grid_for(groups);
  if (y_dtype == TLHIP_F16)
    hipLaunchKernelGGL(epilogue_tail_kernel<_Float16>, dim3(grid), dim3(256), 0, stream, (_Float16*)y, groups, n, ep);
  else
    hipLaunchKernelGGL(epilogue_tail_kernel<float>, dim3(grid), dim3(256), 0, stream, (float*)y, groups, n, ep);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}

}  // namespace tlhip

using namespace tlhip;

extern "C" {

int tlhip_bias_add(const void* in, int dtype, const void* bias, int bias_dtype, void* out, int64_t m, int64_t n,
                   tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (m < 0 || n < 0) return set_error(TLHIP_ERR_INVALID, "bias_add: negative shape");
  const int64_t count = m * n;
  if (count == 0) return TLHIP_OK;
  if (!in || !bias || !out) return set_error(TLHIP_ERR_INVALID, "bias_add: null pointer");
  if ((dtype != TLHIP_F32 && dtype != TLHIP_F16) || (bias_dtype != TLHIP_F32 && bias_dtype != TLHIP_F16))
    return set_error(TLHIP_ERR_INVALID, "bias_add: bad dtype");
  hipStream_t s = resolve_stream(stream);
  if (dtype == TLHIP_F16)
    hipLaunchKernelGGL(bias_add_kernel<_Float16>, dim3(grid_for(count)), dim3(256), 0, s, (const _Float16*)in, bias,
                       bias_dtype, (_Float16*)out, count, n);
  else
    hipLaunchKernelGGL(bias_add_kernel<float>, dim3(grid_for(count)), dim3(256), 0, s, (const float*)in, bias,
                       bias_dtype, (float*)out, count, n);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}

int tlhip_unary(int op, const void* in, int dtype, void* out, int64_t count, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (count < 0) return set_error(TLHIP_ERR_INVALID, "unary: negative count");
  if (count == 0) return TLHIP_OK;
  if (!in || !out) return set_error(TLHIP_ERR_INVALID, "unary: null pointer");
  if (op < TLHIP_UNARY_NONE || op > TLHIP_UNARY_TANH) return set_error(TLHIP_ERR_INVALID, "unary: unknown op %d", op);
  if (dtype != TLHIP_F32 && dtype != TLHIP_F16) return set_error(TLHIP_ERR_INVALID, "unary: bad dtype");
  hipStream_t s = resolve_stream(stream);
  if (dtype == TLHIP_F16)
    hipLaunchKernelGGL(unary_kernel<_Float16>, dim3(grid_for(count)), dim3(256), 0, s, op, (const _Float16*)in,
                       (_Float16*)out, count);
  else
    hipLaunchKernelGGL(unary_kernel<float>, dim3(grid_for(count)), dim3(256), 0, s, op, (const float*)in,
                       (float*)out, count);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}

int tlhip_gated_mul(int unary, const void* gate, const void* up, int dtype, void* out, int64_t count,
                    tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (count < 0) return set_error(TLHIP_ERR_INVALID, "gated_mul: negative count");
  if (count == 0) return TLHIP_OK;
  if (!gate || !up || !out) return set_error(TLHIP_ERR_INVALID, "gated_mul: null pointer");
  if (unary < TLHIP_UNARY_NONE || unary > TLHIP_UNARY_TANH)
    return set_error(TLHIP_ERR_INVALID, "gated_mul: unknown op %d", unary);
  if (dtype != TLHIP_F32 && dtype != TLHIP_F16) return set_error(TLHIP_ERR_INVALID, "gated_mul: bad dtype");
  hipStream_t s = resolve_stream(stream);
  if (dtype == TLHIP_F16)
    hipLaunchKernelGGL(gated_mul_kernel<_Float16>, dim3(grid_for(count)), dim3(256), 0, s, unary,
                       (const _Float16*)gate, (const _Float16*)up, (_Float16*)out, count);
  else
    hipLaunchKernelGGL(gated_mul_kernel<float>, dim3(grid_for(count)), dim3(256), 0, s, unary, (const float*)gate,
                       (const float*)up, (float*)out, count);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}

int tlhip_rmsnorm(const void* x, int x_dtype, const float* weight, void* y, int y_dtype, int64_t m, int64_t d,
                  float eps, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (m < 0 || d < 0) return set_error(TLHIP_ERR_INVALID, "rmsnorm: negative shape");
  if (m == 0 || d == 0) return TLHIP_OK;
  if (!x || !weight || !y) return set_error(TLHIP_ERR_INVALID, "rmsnorm: null pointer");
  if ((x_dtype != TLHIP_F32 && x_dtype != TLHIP_F16) || (y_dtype != TLHIP_F32 && y_dtype != TLHIP_F16))
    return set_error(TLHIP_ERR_INVALID, "rmsnorm: bad dtype");
  if (!(eps >= 0.f)) return set_error(TLHIP_ERR_INVALID, "rmsnorm: eps must be >= 0");
  if (m > 0x7fffffff) return set_error(TLHIP_ERR_INVALID, "rmsnorm: too many rows");
  hipStream_t s = resolve_stream(stream);
  const dim3 grid((unsigned)m), block(256);
  if (x_dtype == TLHIP_F16 && y_dtype == TLHIP_F16)
    hipLaunchKernelGGL((rmsnorm_kernel<_Float16, _Float16>), grid, block, 0, s, (const _Float16*)x, weight,
                       (_Float16*)y, d, eps);
  else if (x_dtype == TLHIP_F16)
    hipLaunchKernelGGL((rmsnorm_kernel<_Float16, float>), grid, block, 0, s, (const _Float16*)x, weight, (float*)y, d,
                       eps);
  else if (y_dtype == TLHIP_F16)
    hipLaunchKernelGGL((rmsnorm_kernel<float, _Float16>), grid, block, 0, s, (const float*)x, weight, (_Float16*)y, d,
                       eps);
  else
    hipLaunchKernelGGL((rmsnorm_kernel<float, float>), grid, block, 0, s, (const float*)x, weight, (float*)y, d, eps);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}

int tlhip_cast(const void* in, int in_dtype, void* out, int out_dtype, int64_t count, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (count < 0) return set_error(TLHIP_ERR_INVALID, "cast: negative count");
  if (count == 0) return TLHIP_OK;
  if (!in || !out) return set_error(TLHIP_ERR_INVALID, "cast: null pointer");
  hipStream_t s = resolve_stream(stream);
  if (in_dtype == TLHIP_F32 && out_dtype == TLHIP_F16)
    hipLaunchKernelGGL((cast_kernel<float, _Float16>), dim3(grid_for(count)), dim3(256), 0, s, (const float*)in,
                       (_Float16*)out, count);
  else if (in_dtype == TLHIP_F16 && out_dtype == TLHIP_F32)
    hipLaunchKernelGGL((cast_kernel<_Float16, float>), dim3(grid_for(count)), dim3(256), 0, s, (const _Float16*)in,
                       (float*)out, count);
  else if (in_dtype == out_dtype && (in_dtype == TLHIP_F32 || in_dtype == TLHIP_F16))
    TLHIP_CHECK_HIP(hipMemcpyAsync(out, in, (size_t)count * (in_dtype == TLHIP_F16 ? 2 : 4), hipMemcpyDeviceToDevice, s));
  else
    return set_error(TLHIP_ERR_INVALID, "cast: unsupported dtypes %d -> %d", in_dtype, out_dtype);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}

}  // extern "C"
