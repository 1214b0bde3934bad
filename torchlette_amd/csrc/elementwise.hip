// The three small ops that sit either side of the packed matmul when the
// frontend calls them unfused (api.linear issues matmul, then add —
// src/frontend/torchlette.ts:887-894 — and the model issues the activation):
// bias add over the last dimension, a unary activation, and an f32<->f16 cast.
// All are one pass over the data, 16 bytes per lane where alignment allows.
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

int grid_for(int64_t count) {
  const int64_t blocks = (count + 255) / 256;
  const int64_t cap = (int64_t)device_cu_count() * 16;
  return (int)std::max<int64_t>(1, std::min(blocks, cap));
}

}  // namespace
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
