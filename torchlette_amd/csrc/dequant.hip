// Explicit dequantisation of a packed weight to f32 [N,K], bit-exact against
// the reference's host dequantizeToF32 (src/backend/quantize.ts:138-156).
//
// HBM-bound: 4 output bytes per weight against 1 (int8) or 0.5 (int4) input
// bytes, so each lane turns one 16-byte load into four (int8) or eight (int4)
// 16-byte stores; consecutive lanes take consecutive 16-byte input chunks, so
// both sides are fully coalesced.
//
// INT8_GROUPED: the reference computes (q/127)*scale in double and rounds once
// to f32.  q/127 has only 256 possible values; they are computed once on the
// host with the same IEEE double division and kept in __constant__ memory, so
// the kernel does one double multiply (correctly rounded on the device) and one
// double->float conversion (round to nearest even) per weight.
// INT8_ROW / INT4_GROUPED: q*s has at most 32 resp. 15 significant bits; one
// f32 multiply is the correctly rounded product the definition asks for.
#include "common.h"

namespace tlhip {
namespace {

__constant__ double c_q_over_127[256];  // indexed by the raw byte (two's complement)

__device__ __forceinline__ double f16_bits_to_f64(uint32_t h) {
  // Exact decoding, subnormals and inf/NaN included (quantize.ts:50-60).
  const uint32_t e = (h >> 10) & 0x1fu, f = h & 0x3ffu;
  double v;
  if (e == 0) {
    v = ldexp((double)f, -24);
  } else if (e == 31) {
    v = f ? __longlong_as_double(0x7ff8000000000000LL) : __longlong_as_double(0x7ff0000000000000LL);
  } else {
    v = ldexp((double)(1024u + f), (int)e - 25);
  }
  return (h & 0x8000u) ? -v : v;
}

__device__ __forceinline__ float f16_bits_to_f32(uint32_t h) {
  return (float)f16_bits_to_f64(h);  // exact: every f16 is an f32
}

// One lane = one 16-byte chunk of packed words = 16 int8 weights.
__global__ __launch_bounds__(256) void dequant_int8_grouped_kernel(const uint4* __restrict__ packed,
                                                                  const uint16_t* __restrict__ scales,
                                                                  float4* __restrict__ out, int64_t n_chunks,
                                                                  int chunks_per_row, int chunks_per_group,
                                                                  int groups_per_row) {
  int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; c < n_chunks; c += stride) {
    const int64_t row = c / chunks_per_row;
    const int cr = (int)(c - row * chunks_per_row);
    const double s = f16_bits_to_f64(scales[row * groups_per_row + cr / chunks_per_group]);
    const uint4 w = packed[c];
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4 o;
      o.x = (float)(c_q_over_127[words[i] & 0xffu] * s);
      o.y = (float)(c_q_over_127[(words[i] >> 8) & 0xffu] * s);
      o.z = (float)(c_q_over_127[(words[i] >> 16) & 0xffu] * s);
      o.w = (float)(c_q_over_127[words[i] >> 24] * s);
      out[c * 4 + i] = o;
    }
  }
}

__global__ __launch_bounds__(256) void dequant_int8_row_kernel(const uint4* __restrict__ packed,
                                                              const float* __restrict__ row_scales,
                                                              float4* __restrict__ out, int64_t n_chunks,
                                                              int chunks_per_row) {
  int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; c < n_chunks; c += stride) {
    const int64_t row = c / chunks_per_row;
    const float s = row_scales[row];
    const uint4 w = packed[c];
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float4 o;
      o.x = (float)(int8_t)(words[i] & 0xffu) * s;
      o.y = (float)(int8_t)((words[i] >> 8) & 0xffu) * s;
      o.z = (float)(int8_t)((words[i] >> 16) & 0xffu) * s;
      o.w = (float)(int8_t)(words[i] >> 24) * s;
      out[c * 4 + i] = o;
    }
  }
}

// One lane = one 16-byte chunk = 32 int4 weights.
__global__ __launch_bounds__(256) void dequant_int4_grouped_kernel(const uint4* __restrict__ packed,
                                                                  const uint16_t* __restrict__ scales,
                                                                  float4* __restrict__ out, int64_t n_chunks,
                                                                  int chunks_per_row, int group_size,
                                                                  int groups_per_row) {
  int64_t c = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; c < n_chunks; c += stride) {
    const int64_t row = c / chunks_per_row;
    const int cr = (int)(c - row * chunks_per_row);
    const uint16_t* srow = scales + row * groups_per_row;
    const uint4 w = packed[c];
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      // 8 weights of one word share a group whenever group_size % 8 == 0.
      const int k0 = cr * 32 + i * 8;
      const float s = f16_bits_to_f32(srow[k0 / group_size]);
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int q = ((int)(words[i] << (28 - 4 * j))) >> 28;  // sign-extend nibble j
        v[j] = (float)q * s;
      }
      out[c * 8 + i * 2] = make_float4(v[0], v[1], v[2], v[3]);
      out[c * 8 + i * 2 + 1] = make_float4(v[4], v[5], v[6], v[7]);
    }
  }
}

// Generic fallbacks for shapes whose rows are not whole 16-byte chunks
// (K % 16 != 0 for int8, K % 32 != 0 for int4): one lane per packed word.
__global__ __launch_bounds__(256) void dequant_word_kernel(int format, const uint32_t* __restrict__ packed,
                                                          const void* __restrict__ scales,
                                                          float* __restrict__ out, int64_t n_words,
                                                          int words_per_row, int group_size,
                                                          int groups_per_row) {
  int64_t wi = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  for (; wi < n_words; wi += stride) {
    const int64_t row = wi / words_per_row;
    const int wr = (int)(wi - row * words_per_row);
    const uint32_t word = packed[wi];
    if (format == TLHIP_FMT_INT4_GROUPED) {
      const uint16_t* srow = (const uint16_t*)scales + row * groups_per_row;
      for (int j = 0; j < 8; ++j) {
        const int kk = wr * 8 + j;
        const int q = ((int)(word << (28 - 4 * j))) >> 28;
        out[wi * 8 + j] = (float)q * f16_bits_to_f32(srow[kk / group_size]);
      }
    } else if (format == TLHIP_FMT_INT8_ROW) {
      const float s = ((const float*)scales)[row];
      for (int j = 0; j < 4; ++j) out[wi * 4 + j] = (float)(int8_t)((word >> (8 * j)) & 0xffu) * s;
    } else {
      const uint16_t* srow = (const uint16_t*)scales + row * groups_per_row;
      for (int j = 0; j < 4; ++j) {
        const int kk = wr * 4 + j;
        const double s = f16_bits_to_f64(srow[kk / group_size]);
        out[wi * 4 + j] = (float)(c_q_over_127[(word >> (8 * j)) & 0xffu] * s);
      }
    }
  }
}

bool g_table_ready = false;

int ensure_table() {
  if (g_table_ready) return TLHIP_OK;
  double t[256];
  for (int b = 0; b < 256; ++b) {
    const int q = b >= 128 ? b - 256 : b;
    // volatile keeps the host compiler from folding this into a multiply by a reciprocal
    volatile double num = (double)q, den = 127.0;
    t[b] = num / den;
  }
  TLHIP_CHECK_HIP(hipMemcpyToSymbol(HIP_SYMBOL(c_q_over_127), t, sizeof(t)));
  g_table_ready = true;
  return TLHIP_OK;
}

int grid_for(int64_t items, int cus) {
  const int64_t blocks = (items + 255) / 256;
  const int64_t cap = (int64_t)cus * 16;
  return (int)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

}  // namespace

int launch_dequant(const tlhip_qweight_t& w, float* out, hipStream_t stream) {
  const int64_t n = w.n, k = w.k;
  if (n == 0 || k == 0) return TLHIP_OK;
  const int cus = device_cu_count();
  const int g = w.group_size;
  if (w.format == TLHIP_FMT_INT8_GROUPED) {
    int rc = ensure_table();
    if (rc) return rc;
  }
  if (w.format == TLHIP_FMT_INT4_GROUPED) {
    if (k % 32 == 0 && g % 8 == 0) {
      const int64_t chunks = n * (k / 32);
      hipLaunchKernelGGL(dequant_int4_grouped_kernel, dim3(grid_for(chunks, cus)), dim3(256), 0, stream,
                         (const uint4*)w.packed, (const uint16_t*)w.scales, (float4*)out, chunks,
                         (int)(k / 32), g, (int)(k / g));
    } else {
      const int64_t words = n * (k / 8);
      hipLaunchKernelGGL(dequant_word_kernel, dim3(grid_for(words, cus)), dim3(256), 0, stream, w.format,
                         (const uint32_t*)w.packed, w.scales, out, words, (int)(k / 8), g, (int)(k / g));
    }
  } else if (w.format == TLHIP_FMT_INT8_ROW) {
    if (k % 16 == 0) {
      const int64_t chunks = n * (k / 16);
      hipLaunchKernelGGL(dequant_int8_row_kernel, dim3(grid_for(chunks, cus)), dim3(256), 0, stream,
                         (const uint4*)w.packed, (const float*)w.scales, (float4*)out, chunks, (int)(k / 16));
    } else {
      const int64_t words = n * (k / 4);
      hipLaunchKernelGGL(dequant_word_kernel, dim3(grid_for(words, cus)), dim3(256), 0, stream, w.format,
                         (const uint32_t*)w.packed, w.scales, out, words, (int)(k / 4), 0, 0);
    }
  } else {
    if (k % 16 == 0 && g % 16 == 0) {
      const int64_t chunks = n * (k / 16);
      hipLaunchKernelGGL(dequant_int8_grouped_kernel, dim3(grid_for(chunks, cus)), dim3(256), 0, stream,
                         (const uint4*)w.packed, (const uint16_t*)w.scales, (float4*)out, chunks,
                         (int)(k / 16), g / 16, (int)(k / g));
    } else {
      const int64_t words = n * (k / 4);
      hipLaunchKernelGGL(dequant_word_kernel, dim3(grid_for(words, cus)), dim3(256), 0, stream, w.format,
                         (const uint32_t*)w.packed, w.scales, out, words, (int)(k / 4), g, (int)(k / g));
    }
  }
  TLHIP_CHECK_HIP(hipGetLastError());
  count_dequant_dispatch();
  return TLHIP_OK;
}

}  // namespace tlhip
