// Top-k of one logits row on the device, so that the 256 000 logits the LM-head
// GEMV produces are never read back (the reference's sampling prefilter,
// src/backend/webgpu/topk-kernel.ts:1-30; readTopK / deviceTopK,
// src/backend/types.ts:632-634, 669-678).  Result: the k largest values in
// descending order, ties broken towards the smaller index (what a linear scan that
// keeps the first maximum gives), as (value, index) pairs.
//
// Every element becomes a 64-bit key, (order-preserving bits of the value) << 32 |
// (0xffffffff - index), so that "larger key" is exactly "larger value, then smaller
// index"; NaN maps below every number.  A workgroup sorts up to 4096 keys in LDS
// (bitonic, descending) and keeps the first k; levels repeat (chunk -> k per
// workgroup) until one workgroup holds the answer.  Chunks of 1024 keys for
// k <= 256 (many small sorts, every CU busy: 250 + 16 + 1 workgroups for 256 000
// logits at k = 64), of 4096 above.  HBM traffic: the row once.
#include "device_utils.h"

namespace tlhip {
namespace {

constexpr float kTopkNegInf = -3.4028234e38f;  // the reference's filler for missing entries

__device__ __forceinline__ uint64_t topk_key(float v, uint32_t index) {
  const uint32_t b = __builtin_bit_cast(uint32_t, v);
  uint32_t k = (b & 0x80000000u) ? ~b : (b | 0x80000000u);
  if (v != v) k = 0u;  // NaN: below everything
  return ((uint64_t)k << 32) | (uint64_t)(0xffffffffu - index);
}

__device__ __forceinline__ float topk_value(uint64_t key) {
  const uint32_t k = (uint32_t)(key >> 32);
  const uint32_t b = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __builtin_bit_cast(float, b);
}

// FROM_FLOAT: keys are made from `logits[offset + i]` with index i; else read from `keys_in`.
// The first `k` keys of the sorted chunk go to keys_out[block * k ..]; with `final`
// they are decoded into values / indices instead.
template <bool FROM_FLOAT, int kTopkChunk>
__global__ __launch_bounds__(kTopkChunk / 4) void topk_level_kernel(const float* __restrict__ logits, int64_t offset,
                                                        const uint64_t* __restrict__ keys_in, int64_t count, int k,
                                                        uint64_t* __restrict__ keys_out, int final,
                                                        float* __restrict__ out_values,
                                                        void* __restrict__ out_indices, int index_dtype) {
  __shared__ uint64_t keys[kTopkChunk];
  const int64_t base = (int64_t)blockIdx.x * kTopkChunk;
  constexpr int THREADS = kTopkChunk / 4;
#pragma unroll
  for (int i = threadIdx.x; i < kTopkChunk; i += THREADS) {
    const int64_t e = base + i;
    uint64_t key = 0;  // padding sorts last: the index part of a real key is at least 1
    if (e < count) key = FROM_FLOAT ? topk_key(logits[offset + e], (uint32_t)e) : keys_in[e];
    keys[i] = key;
  }
  __syncthreads();
  // bitonic sort, descending
  for (int size = 2; size <= kTopkChunk; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      // two compare-exchanges per thread, both pairs read before either is written
      const int t0 = threadIdx.x, t1 = threadIdx.x + THREADS;
      const int lo0 = 2 * t0 - (t0 & (stride - 1)), lo1 = 2 * t1 - (t1 & (stride - 1));
      const uint64_t a0 = keys[lo0], b0 = keys[lo0 + stride], a1 = keys[lo1], b1 = keys[lo1 + stride];
      const bool swap0 = (a0 < b0) == ((lo0 & size) == 0), swap1 = (a1 < b1) == ((lo1 & size) == 0);
      keys[lo0] = swap0 ? b0 : a0;
      keys[lo0 + stride] = swap0 ? a0 : b0;
      keys[lo1] = swap1 ? b1 : a1;
      keys[lo1 + stride] = swap1 ? a1 : b1;
      __syncthreads();
    }
  }
  for (int i = threadIdx.x; i < k; i += THREADS) {
    const uint64_t key = keys[i];
    if (final) {
      const bool real = key != 0;
      out_values[i] = real ? topk_value(key) : kTopkNegInf;
      const int32_t idx = real ? (int32_t)(0xffffffffu - (uint32_t)key) : -1;
      if (index_dtype == TLHIP_F32) ((float*)out_indices)[i] = (float)idx;  // token ids as f32 (deviceTopK)
      else ((int32_t*)out_indices)[i] = idx;
    } else {
      keys_out[(int64_t)blockIdx.x * k + i] = key;
    }
  }
}

}  // namespace
}  // namespace tlhip

using namespace tlhip;

extern "C" int tlhip_topk(const float* logits, int64_t offset, int64_t length, int k, float* out_values,
                          void* out_indices, int index_dtype, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (k < 1 || k > 1024) return set_error(TLHIP_ERR_INVALID, "topk: k=%d must be 1..1024", k);
  if (index_dtype != TLHIP_F32 && index_dtype != TLHIP_I32)
    return set_error(TLHIP_ERR_INVALID, "topk: indices are TLHIP_I32 or TLHIP_F32");
  if (offset < 0 || length < 0) return set_error(TLHIP_ERR_INVALID, "topk: negative offset or length");
  if (length > (int64_t)0xfffffffe) return set_error(TLHIP_ERR_INVALID, "topk: length above 2^32-2");
  if (!out_values || !out_indices || (length > 0 && !logits)) return set_error(TLHIP_ERR_INVALID, "topk: null pointer");
  hipStream_t s = resolve_stream(stream);
  // level 0 reads the floats; later levels read the keys the level before wrote
  // into the stream's workspace, alternating between its two halves
  const int chunk = k <= 256 ? 1024 : 4096;
  int64_t count = length;
  int64_t blocks = (count + chunk - 1) / chunk;
  if (blocks < 1) blocks = 1;
  float* ws = nullptr;
  int* counters = nullptr;
  const size_t half = kSplitWorkspaceFloats / 4;  // uint64 keys per half
  if (blocks > 1) {
    if ((size_t)blocks * k > half)
      return set_error(TLHIP_ERR_INVALID, "topk: length %lld with k=%d needs more workspace than the library holds",
                       (long long)length, k);
    const int rc = split_workspace(s, &ws, &counters);
    if (rc) return rc;
  }
  uint64_t* bufs[2] = {(uint64_t*)ws, (uint64_t*)ws + half};
  int level = 0;
  const uint64_t* keys_in = nullptr;
  while (true) {
    const int final = blocks == 1;
    uint64_t* keys_out = final ? nullptr : bufs[level & 1];
    const dim3 grid((unsigned)blocks), threads(chunk / 4);
    const int64_t zero = 0;
    if (level == 0 && chunk == 1024)
      hipLaunchKernelGGL((topk_level_kernel<true, 1024>), grid, threads, 0, s, logits, offset, nullptr, count, k,
                         keys_out, final, out_values, out_indices, index_dtype);
    else if (level == 0)
      hipLaunchKernelGGL((topk_level_kernel<true, 4096>), grid, threads, 0, s, logits, offset, nullptr, count, k,
                         keys_out, final, out_values, out_indices, index_dtype);
    else if (chunk == 1024)
      hipLaunchKernelGGL((topk_level_kernel<false, 1024>), grid, threads, 0, s, nullptr, zero, keys_in, count, k,
                         keys_out, final, out_values, out_indices, index_dtype);
    else
      hipLaunchKernelGGL((topk_level_kernel<false, 4096>), grid, threads, 0, s, nullptr, zero, keys_in, count, k,
                         keys_out, final, out_values, out_indices, index_dtype);
    TLHIP_CHECK_HIP(hipGetLastError());
    if (final) break;
    keys_in = keys_out;
    count = blocks * k;
    blocks = (count + chunk - 1) / chunk;
    ++level;
  }
  return TLHIP_OK;
}
