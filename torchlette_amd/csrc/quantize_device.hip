// quantizeLinearWeight (src/backend/quantize.ts:77-131) on the device, for
// quantize-at-load of weights that are already resident: same bits as the host
// routine for every input (f64 arithmetic for the scale reciprocal and the
// product, Math.round ties toward +infinity, the reference's f16 encoder with
// its round-half-up subnormals).
//
// One workgroup per weight row at a time.  Pass 1: each thread takes 16-byte
// pieces (4 weights = one packed word) and folds |w| into the group's maximum in
// LDS with an unsigned atomic max on the float bits (non-negative floats order
// like their bit patterns; NaN is skipped, as `a > max` is false for NaN in the
// reference).  Pass 2: scale bits from the maximum, then the packed words.
// HBM-bound: 4 bytes read (twice; the second read hits L2) and 1 + 2/G written
// per weight.
#include "device_utils.h"

namespace tlhip {
namespace {

// quantize.ts:22-47
__device__ __forceinline__ uint32_t encode_f16_ref(float v) {
  const uint32_t u = __builtin_bit_cast(uint32_t, v);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const int e16 = int((u >> 23) & 0xffu) - 112;
  const uint32_t frac = u & 0x007fffffu;
  if (e16 >= 31) return sign | 0x7c00u;
  if (e16 >= 1) {
    uint32_t h = sign | (uint32_t(e16) << 10) | (frac >> 13);
    const uint32_t rem = frac & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h += 1;
    return h;
  }
  if (e16 < -10) return sign;
  const uint32_t shifted = (frac | 0x00800000u) >> uint32_t(1 - e16);
  return sign | ((shifted >> 13) + ((shifted >> 12) & 1u));
}

// quantize.ts:50-60 for a non-negative pattern; exact in double
__device__ __forceinline__ double decode_f16_ref(uint32_t h) {
  const int e = (h >> 10) & 0x1f;
  const int f = h & 0x3ff;
  if (e == 0) return ldexp((double)f, -24);
  if (e == 31) return f ? __builtin_nan("") : __builtin_inf();
  return ldexp((double)(1024 + f), e - 25);
}

__device__ __forceinline__ uint32_t quantize_one(float w, double inv) {
  const double t = (double)w * inv;
  int q = 0;  // NaN -> 0 (NaN & 0xff in JavaScript)
  if (t == t) {
    double rr = t;
    if (!__builtin_isinf(t)) {
      const double f = floor(t);
      rr = (t - f >= 0.5) ? f + 1.0 : f;  // Math.round
    }
    q = rr > 127.0 ? 127 : (rr < -127.0 ? -127 : (int)rr);
  }
  return (uint32_t)q & 0xffu;
}

__global__ __launch_bounds__(256) void quantize_int8_grouped_kernel(const float* __restrict__ w, int64_t n, int k,
                                                                   int g, uint32_t* __restrict__ packed,
                                                                   uint16_t* __restrict__ scales) {
  extern __shared__ uint32_t amax_bits[];  // one per group of the row
  const int groups = k / g, words = k / 4;
  for (int64_t row = blockIdx.x; row < n; row += gridDim.x) {
    const float4_t* wr = (const float4_t*)(w + row * k);
    for (int i = threadIdx.x; i < groups; i += blockDim.x) amax_bits[i] = 0u;
    __syncthreads();
    for (int i = threadIdx.x; i < words; i += blockDim.x) {
      const float4_t v = wr[i];
      float m = 0.f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float a = fabsf(v[e]);
        if (a > m) m = a;  // false for NaN
      }
      // a word never straddles two groups: g is a multiple of 4
      atomicMax(&amax_bits[(i * 4) / g], __builtin_bit_cast(uint32_t, m));
    }
    __syncthreads();
    for (int i = threadIdx.x; i < groups; i += blockDim.x)
      scales[row * groups + i] = (uint16_t)encode_f16_ref(__builtin_bit_cast(float, amax_bits[i]));
    for (int i = threadIdx.x; i < words; i += blockDim.x) {
      const uint32_t sbits = encode_f16_ref(__builtin_bit_cast(float, amax_bits[(i * 4) / g]));
      const double s = decode_f16_ref(sbits);
      const double inv = s > 0 ? 127.0 / s : 0.0;
      const float4_t v = wr[i];
      packed[row * words + i] = quantize_one(v[0], inv) | (quantize_one(v[1], inv) << 8) |
                                (quantize_one(v[2], inv) << 16) | (quantize_one(v[3], inv) << 24);
    }
    __syncthreads();  // amax_bits is reused by the next row
  }
}

}  // namespace
}  // namespace tlhip

using namespace tlhip;

extern "C" int tlhip_quantize_int8_grouped_device(const float* weight, int64_t n, int64_t k, int64_t group_size,
                                                  uint32_t* packed, uint16_t* scales, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (n < 0 || k < 0) return set_error(TLHIP_ERR_INVALID, "quantize: negative shape");
  if (k % 4 != 0) return set_error(TLHIP_ERR_INVALID, "quantize: K=%lld must be divisible by 4", (long long)k);
  if (group_size <= 0 || k % group_size != 0)
    return set_error(TLHIP_ERR_INVALID, "quantize: K=%lld must be divisible by groupSize=%lld", (long long)k,
                     (long long)group_size);
  if (group_size % 4 != 0)
    return set_error(TLHIP_ERR_INVALID, "quantize (device): groupSize=%lld must be a multiple of 4",
                     (long long)group_size);
  if (n == 0 || k == 0) return TLHIP_OK;
  if (!weight || !packed || !scales) return set_error(TLHIP_ERR_INVALID, "quantize: null pointer");
  if (((uintptr_t)weight & 15) != 0) return set_error(TLHIP_ERR_INVALID, "quantize: weight must be 16-byte aligned");
  if (k > (1 << 22)) return set_error(TLHIP_ERR_INVALID, "quantize (device): K=%lld above 4194304", (long long)k);
  const size_t lds = (size_t)(k / group_size) * sizeof(uint32_t);
  if (lds > 64 * 1024)
    return set_error(TLHIP_ERR_INVALID, "quantize (device): %lld groups per row do not fit LDS",
                     (long long)(k / group_size));
  const int64_t cap = (int64_t)device_cu_count() * 8;
  const int grid = (int)(n < cap ? n : cap);
  hipLaunchKernelGGL(quantize_int8_grouped_kernel, dim3(grid), dim3(256), lds, resolve_stream(stream), weight, n,
                     (int)k, (int)group_size, packed, scales);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}
