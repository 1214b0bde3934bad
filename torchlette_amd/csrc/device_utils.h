// Device helpers shared by the GEMV and GEMM kernels: the epilogue chain, f16
// scale decoding, int4/int8 unpacking into packed f16 pairs, and lane
// reductions over DPP.
#pragma once

#include "common.h"

namespace tlhip {

typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));

// Reinterpretations take their argument BY VALUE: __builtin_bit_cast applied
// directly to a vector-element lvalue (v.y) reads the vector's first element.
__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ float as_float(uint32_t v) { return __builtin_bit_cast(float, v); }

__device__ __forceinline__ float half_bits_to_float(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}

// ---------------------------------------------------------------- epilogue
// Formulas: relu/silu/sigmoid from src/ops/semantic/catalog.ts:81-109, gelu
// (tanh form) from composite.ts:40-51, gelu_erf with the Abramowitz-Stegun
// polynomial of erf.ts:28-56 — evaluated in f32 as the reference's GPU
// epilogues are (src/schedule/matmul-skeleton.ts:916-966).
// exp and 1/x through the hardware approximations (v_exp_f32 after a scale by
// log2 e, v_rcp_f32: about 1 ulp each) instead of the correctly rounded library
// routines, which cost 10-20 VALU instructions per element: the epilogue runs
// once per output element and is a visible share of a GEMM tile's VALU time.
__device__ __forceinline__ float fast_exp(float v) { return __expf(v); }
__device__ __forceinline__ float fast_rcp(float v) { return __builtin_amdgcn_rcpf(v); }
__device__ __forceinline__ float fast_tanh(float v) {
  // tanh(v) = 1 - 2 / (1 + exp(2v)); exp overflow -> inf -> 1, underflow -> 0 -> -1
  return 1.f - 2.f * fast_rcp(1.f + fast_exp(2.f * v));
}

__device__ __forceinline__ float apply_unary(int op, float v) {
  switch (op) {
    case TLHIP_UNARY_RELU: return v > 0.f ? v : 0.f;
    case TLHIP_UNARY_SILU: return v * fast_rcp(1.f + fast_exp(-v));
    case TLHIP_UNARY_SIGMOID: return fast_rcp(1.f + fast_exp(-v));
    case TLHIP_UNARY_TANH: return fast_tanh(v);
    case TLHIP_UNARY_GELU_TANH:
      return (0.5f * v) * (1.f + fast_tanh(0.7978845608f * (v + 0.044715f * (v * (v * v)))));
    case TLHIP_UNARY_GELU_ERF: {
      const float u = v * 0.70710678118654752f;
      const float ax = fabsf(u);
      const float t = fast_rcp(1.f + 0.3275911f * ax);
      const float poly =
          ((((1.061405429f * t - 1.453152027f) * t + 1.421413741f) * t - 0.284496736f) * t + 0.254829592f) * t;
      const float e = 1.f - poly * fast_exp(-ax * ax);
      return (0.5f * v) * (1.f + (u < 0.f ? -e : e));
    }
    default: return v;
  }
}

// One step of the chain on one value: `col` is the output column n, `idx` the output
// element m*N + n (what a binary step's [M,N] input is indexed by).
__device__ __forceinline__ float apply_epilogue_step(int kind, int op, const void* input, int input_dtype, float v,
                                                     int64_t col, int64_t idx) {
  if (kind == TLHIP_EPI_BIAS || kind == TLHIP_EPI_BINARY) {
    const int64_t at = kind == TLHIP_EPI_BIAS ? col : idx;
    float b;
    if (input_dtype == TLHIP_F16) b = (float)((const _Float16*)input)[at];
    else b = ((const float*)input)[at];
    if (kind == TLHIP_EPI_BIAS || op == TLHIP_BINARY_ADD) return v + b;
    return op == TLHIP_BINARY_SUB ? v - b : v * b;
  }
  if (kind == TLHIP_EPI_UNARY) return apply_unary(op, v);
  if (kind == TLHIP_EPI_CAST_F16) return (float)(_Float16)v;
  return v;
}

// acc*alpha, then the ops in order.
__device__ __forceinline__ float apply_epilogue(const DevEpilogue& ep, float v, int64_t col, int64_t idx) {
  for (int i = 0; i < ep.n_ops; ++i) v = apply_epilogue_step(ep.kind[i], ep.unary[i], ep.input[i], ep.input_dtype[i], v, col, idx);
  return v;
}

// The same on COUNT values of one output column (element_of(j): the output element of
// value j, or -1 for a value that will not be stored): the ops are the outer loop,
// unrolled over the fixed capacity with constant indices, so that the epilogue's fields
// stay in scalar registers however many values the caller holds (a run-time index into
// the kernel arguments makes the compiler copy them to scratch memory).
template <int COUNT, typename ElementOf>
__device__ __forceinline__ void apply_epilogue_all(const DevEpilogue& ep, float (&v)[COUNT], int64_t col, ElementOf element_of) {
#pragma unroll
  for (int i = 0; i < TLHIP_MAX_EPILOGUE_OPS; ++i) {
    if (i < ep.n_ops) {
      if (ep.kind[i] == TLHIP_EPI_BIAS) {
        float b;
        if (ep.input_dtype[i] == TLHIP_F16) b = (float)((const _Float16*)ep.input[i])[col];
        else b = ((const float*)ep.input[i])[col];
#pragma unroll
        for (int j = 0; j < COUNT; ++j) v[j] += b;
      } else if (ep.kind[i] == TLHIP_EPI_UNARY) {
#pragma unroll
        for (int j = 0; j < COUNT; ++j) v[j] = apply_unary(ep.unary[i], v[j]);
      } else if (ep.kind[i] != TLHIP_EPI_NONE) {
#pragma unroll
        for (int j = 0; j < COUNT; ++j) {
          const int64_t idx = element_of(j);
          if (idx >= 0) v[j] = apply_epilogue_step(ep.kind[i], ep.unary[i], ep.input[i], ep.input_dtype[i], v[j], col, idx);
        }
      }
    }
  }
}

// The chain on 8 consecutive columns of one output row (columns col .. col+7, elements idx
// .. idx+7): the ops are the outer loop, unrolled with constant indices, and where `vec`
// holds (all 8 columns exist and N is a multiple of 8) an input that is 16-byte aligned
// comes as one or two 16-byte loads.  (A chain per element, with a 2- or 4-byte load per
// element and step, made the fused residual add of a 2048 x 12288 GEMM cost 141 us.)
__device__ __forceinline__ void apply_epilogue_row8(const DevEpilogue& ep, float (&v)[8], int64_t col, int64_t idx, bool vec,
                                                    int64_t last_col) {
#pragma unroll
  for (int i = 0; i < TLHIP_MAX_EPILOGUE_OPS; ++i) {
    if (i < ep.n_ops) {
      const int kind = ep.kind[i];
      if (kind == TLHIP_EPI_BIAS || kind == TLHIP_EPI_BINARY) {
        const int64_t at = kind == TLHIP_EPI_BIAS ? col : idx;
        const bool f16 = ep.input_dtype[i] == TLHIP_F16;
        float b[8];
        if (vec && (((uintptr_t)ep.input[i] + (size_t)at * (f16 ? 2 : 4)) & 15) == 0) {
          if (f16) {
            const half8_t h = *(const half8_t*)((const _Float16*)ep.input[i] + at);
#pragma unroll
            for (int e = 0; e < 8; ++e) b[e] = (float)h[e];
          } else {
            const float4_t lo = *(const float4_t*)((const float*)ep.input[i] + at);
            const float4_t hi = *(const float4_t*)((const float*)ep.input[i] + at + 4);
            b[0] = lo[0]; b[1] = lo[1]; b[2] = lo[2]; b[3] = lo[3];
            b[4] = hi[0]; b[5] = hi[1]; b[6] = hi[2]; b[7] = hi[3];
          }
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int64_t off = col + e <= last_col ? e : last_col - col;  // past the row's end: the last column again
            b[e] = f16 ? (float)((const _Float16*)ep.input[i])[at + off] : ((const float*)ep.input[i])[at + off];
          }
        }
        const int op = kind == TLHIP_EPI_BIAS ? (int)TLHIP_BINARY_ADD : ep.unary[i];
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = op == TLHIP_BINARY_ADD ? v[e] + b[e] : (op == TLHIP_BINARY_SUB ? v[e] - b[e] : v[e] * b[e]);
      } else if (kind == TLHIP_EPI_UNARY) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = apply_unary(ep.unary[i], v[e]);
      } else if (kind == TLHIP_EPI_CAST_F16) {
#pragma unroll
        for (int e = 0; e < 8; ++e) v[e] = (float)(_Float16)v[e];
      }
    }
  }
}

__device__ __forceinline__ void store_out(void* y, int y_dtype, int64_t idx, float v) {
  if (y_dtype == TLHIP_F16) ((_Float16*)y)[idx] = (_Float16)v;
  else ((float*)y)[idx] = v;
}

// ------------------------------------------------------------------ unpack
// int4: one u32 holds nibbles j=0..7 for k = 8*word + j, two's complement.
// XOR 0x8 turns a nibble into q+8; OR-ing it into the mantissa of 1024.0h
// (0x6400) gives the f16 value 1024+q+8 (or 1024+16*(q+8) for a nibble at bit
// 4), from which q is recovered exactly by one packed add or fma.
// Output order: pairs (k0,k4) (k1,k5) (k2,k6) (k3,k7).
// (a & mask) | orv as the single instruction it is.  Left to itself the compiler
// emits a separate AND and OR for half of the uses (a VOP3 instruction takes no
// 32-bit literal, and it prefers literals to keeping the constants in registers).
__device__ __forceinline__ uint32_t and_or(uint32_t a, uint32_t mask, uint32_t orv) {
  uint32_t d;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(orv));
  return d;
}

__device__ __forceinline__ void unpack_int4_word(uint32_t w, half2_t out[4]) {
  const uint32_t t = w ^ 0x88888888u;
  const uint32_t lo = t, hi = t >> 8;
  const half2_t sub_lo = {(_Float16)-1032.f, (_Float16)-1032.f};  // -(1024 + 8)
  const half2_t mul_hi = {(_Float16)0.0625f, (_Float16)0.0625f};  // 1/16
  const half2_t sub_hi = {(_Float16)-72.f, (_Float16)-72.f};      // -(1024/16 + 8)
  const uint32_t a0 = and_or(lo, 0x000f000fu, 0x64006400u);
  const uint32_t a1 = and_or(lo, 0x00f000f0u, 0x64006400u);
  const uint32_t a2 = and_or(hi, 0x000f000fu, 0x64006400u);
  const uint32_t a3 = and_or(hi, 0x00f000f0u, 0x64006400u);
  out[0] = __builtin_bit_cast(half2_t, a0) + sub_lo;
  out[1] = __builtin_bit_cast(half2_t, a1) * mul_hi + sub_hi;
  out[2] = __builtin_bit_cast(half2_t, a2) + sub_lo;
  out[3] = __builtin_bit_cast(half2_t, a3) * mul_hi + sub_hi;
}

// The matching order for activations: 8 consecutive f16 (one 16-byte load)
// rearranged to (x0,x4) (x1,x5) (x2,x6) (x3,x7).
__device__ __forceinline__ u32x4 permute_x_for_int4(u32x4 v) {
  u32x4 r;
  r.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);  // lo16(x) | lo16(z) << 16 : (x0, x4)
  r.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);  // hi16(x) | hi16(z) << 16 : (x1, x5)
  r.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);  // (x2, x6)
  r.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);  // (x3, x7)
  return r;
}

// int8: bytes b0..b3 hold k = 4*word + 0..3.  XOR 0x80 gives q+128; placed in
// the low mantissa byte of 1024.0h it reads 1024+q+128.  Natural pair order.
__device__ __forceinline__ void unpack_int8_word(uint32_t w, half2_t out[2]) {
  const uint32_t t = w ^ 0x80808080u;
  const half2_t sub = {(_Float16)-1152.f, (_Float16)-1152.f};
  // v_perm_b32 selects bytes from {src0 (bytes 7..4), src1 (bytes 3..0)}
  const uint32_t a0 = __builtin_amdgcn_perm(0x64646464u, t, 0x04010400u);  // 0x64,b1,0x64,b0
  const uint32_t a1 = __builtin_amdgcn_perm(0x64646464u, t, 0x04030402u);  // 0x64,b3,0x64,b2
  out[0] = __builtin_bit_cast(half2_t, a0) + sub;
  out[1] = __builtin_bit_cast(half2_t, a1) + sub;
}

// One 16-byte unit of activations as floats and back (f16: one rounding).
template <typename XT>
__device__ __forceinline__ void unit_to_floats(u32x4 v, float (&f)[16 / sizeof(XT)]) {
  if constexpr (sizeof(XT) == 2) {
    const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const half2_t h = as_half2(w[i]);
      f[2 * i] = (float)h[0];
      f[2 * i + 1] = (float)h[1];
    }
  } else {
    f[0] = as_float(v.x);
    f[1] = as_float(v.y);
    f[2] = as_float(v.z);
    f[3] = as_float(v.w);
  }
}
template <typename XT>
__device__ __forceinline__ u32x4 floats_to_unit(const float (&f)[16 / sizeof(XT)]) {
  u32x4 v;
  if constexpr (sizeof(XT) == 2) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const half2_t h = {(_Float16)f[2 * i], (_Float16)f[2 * i + 1]};
      w[i] = __builtin_bit_cast(uint32_t, h);
    }
    v = (u32x4){w[0], w[1], w[2], w[3]};
  } else {
    v = (u32x4){__builtin_bit_cast(uint32_t, f[0]), __builtin_bit_cast(uint32_t, f[1]),
                __builtin_bit_cast(uint32_t, f[2]), __builtin_bit_cast(uint32_t, f[3])};
  }
  return v;
}

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits
// for every outstanding global load of the wave (vmcnt(0)), which would drain
// the weight loads that were deliberately issued ahead; here only the wave's
// own LDS operations are waited for (lgkmcnt(0)) before s_barrier.
// s_waitcnt immediate on gfx9: vmcnt = 63 (no wait), expcnt = 7 (no wait), lgkmcnt = 0.
__device__ __forceinline__ void lds_barrier() {
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_s_barrier();
}

// ------------------------------------------------------------- reductions
template <int CTRL>
__device__ __forceinline__ float dpp_add(float v) {
  const int moved = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true);
  return v + __builtin_bit_cast(float, moved);
}

// Sum over groups of `lanes` consecutive lanes (16, 32 or 64); every lane of a
// group ends with the group's sum.
__device__ __forceinline__ float group_sum(float v, int lanes) {
  v = dpp_add<0xB1>(v);   // quad_perm [1,0,3,2]
  v = dpp_add<0x4E>(v);   // quad_perm [2,3,0,1]
  v = dpp_add<0x141>(v);  // row_half_mirror
  v = dpp_add<0x140>(v);  // row_mirror
  if (lanes >= 32) v += __shfl_xor(v, 16);
  if (lanes >= 64) v += __shfl_xor(v, 32);
  return v;
}

}  // namespace tlhip
