/*
 * TEST INFRASTRUCTURE — NOT PRODUCT CODE.
 *
 * CPU restatement, in plain C, of torchlette's quantized-weight linear path as
 * its own CPU code computes it.  Only tests, the smoke check and the bench's
 * cpu_baseline leg may load this library; the shipped HIP path never does.
 *
 * Every function cites the reference file:line it follows (paths relative to
 * the torchlette source tree).  JavaScript numbers are IEEE-754 doubles, so a
 * C double with contraction disabled (-ffp-contract=off) performs the same
 * arithmetic; Float32Array stores are (float) casts (round-to-nearest-even).
 *
 * How each function is pinned (see tests/test_oracle_*.py):
 *   ref_f16_bits_to_f32      all 65 536 patterns vs numpy float16 decoding
 *   ref_f32_to_f16_bits      numpy astype(float16) on every normal result;
 *                            closed form floor(|x|*2^24 + 1/2) on the whole
 *                            subnormal range; hand cases for inf/NaN/underflow
 *   ref_quantize_int8_grouped  invariants, half-integer rounding cases, tiny
 *                            hand-worked groups, exact-rational bounds
 *   ref_dequant_*            exact rational arithmetic (fractions.Fraction)
 *                            and numpy float64 over the full (q, scale) table
 *   ref_matmul_nt            the reference's own known answers
 *                            (test/numeric.spec.ts:102-152) and numpy float64
 *   ref_bias_add, ref_unary  the formulas written out in
 *                            test/webgpu/matmul-epilogue.spec.ts:49-75; libm
 *                            exp/tanh stand in for V8's Math.exp/Math.tanh
 *                            (both < 1 ulp in double; the last double bit is
 *                            "parity unpinned", far below the 1e-3 gate)
 *   ref_rmsnorm              the rows and closed form of the reference's own test
 *                            (test/nn-rmsnorm.spec.ts:10-41), unit RMS of the
 *                            output, invariance under scaling of x, constant rows
 *   ref_mul                  numpy float32 multiply (bit-exact)
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

/* ------------------------------------------------------------------ A1 */

/* src/backend/quantize.ts:22-47  f32ToF16Bits.
 * Normal results round to nearest even; results in the f16 subnormal range
 * add bit 12 of the truncated significand (round-half-UP); |x| < 2^-25 gives a
 * signed zero; exponent >= 0x1f (overflow, inf AND NaN) gives signed 0x7c00. */
uint16_t ref_f32_to_f16_bits(float val) {
  uint32_t x;
  memcpy(&x, &val, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  int32_t exp = (int32_t)((x >> 23) & 0xffu) - 127 + 15;
  uint32_t mant = x & 0x7fffffu;
  if (exp <= 0) {
    if (exp < -10) return (uint16_t)sign;
    uint32_t m = (mant | 0x800000u) >> (uint32_t)(1 - exp);
    uint32_t round = (m & 0x1000u) != 0 ? 1u : 0u;
    return (uint16_t)((sign | ((m >> 13) + round)) & 0xffffu);
  }
  if (exp >= 0x1f) return (uint16_t)(sign | 0x7c00u);
  uint32_t half_mant = mant >> 13;
  uint32_t remainder = mant & 0x1fffu;
  uint32_t out = sign | ((uint32_t)exp << 10) | half_mant;
  if (remainder > 0x1000u || (remainder == 0x1000u && (half_mant & 1u) == 1u)) {
    out += 1;
  }
  return (uint16_t)(out & 0xffffu);
}

/* src/backend/quantize.ts:50-60  f16BitsToF32 (returns a JS number: double). */
double ref_f16_bits_to_f64(uint16_t bits) {
  int sign = (bits >> 15) & 0x1;
  int exp = (bits >> 10) & 0x1f;
  int frac = bits & 0x3ff;
  if (exp == 0) {
    if (frac == 0) return sign ? -0.0 : 0.0;
    return (sign ? -1.0 : 1.0) * ldexp(1.0, -14) * ((double)frac / 1024.0);
  }
  if (exp == 31) return frac == 0 ? (sign ? -INFINITY : INFINITY) : NAN;
  return (sign ? -1.0 : 1.0) * ldexp(1.0, exp - 15) * (1.0 + (double)frac / 1024.0);
}

float ref_f16_bits_to_f32(uint16_t bits) { return (float)ref_f16_bits_to_f64(bits); }

void ref_f32_to_f16_bits_array(const float* in, uint16_t* out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = ref_f32_to_f16_bits(in[i]);
}

void ref_f16_bits_to_f32_array(const uint16_t* in, float* out, int64_t n) {
  for (int64_t i = 0; i < n; i++) out[i] = ref_f16_bits_to_f32(in[i]);
}

/* ------------------------------------------------------------------ A2 */

/* ECMAScript Math.round: nearest integer, ties toward +infinity.  Written as
 * floor + exact fractional test so that 0.49999999999999994 and |x| >= 2^52
 * behave as in JavaScript (x + 0.5 would round up wrongly there). */
static double js_math_round(double x) {
  if (isnan(x) || isinf(x)) return x;
  double r = floor(x);
  if (x - r >= 0.5) r += 1.0;
  return r;
}

/* src/backend/quantize.ts:77-131  quantizeLinearWeight.
 * Returns 0 on success; 1, 2, 3 for the three argument errors the reference
 * throws on (length is the caller's business here; k%4; k%group).
 * NaN weights never raise absMax (the `a > absMax` test is false) and quantize
 * to 0 (NaN & 0xff == 0 in JS); an infinite absMax gives scale=inf, inv=0. */
int ref_quantize_int8_grouped(const float* weight, int64_t n, int64_t k, int64_t group_size,
                              uint32_t* packed, uint16_t* scales) {
  if (k % 4 != 0) return 2;
  if (group_size <= 0 || k % group_size != 0) return 3;
  int64_t groups_per_row = k / group_size;
  int64_t words_per_row = k / 4;
  memset(packed, 0, (size_t)(n * words_per_row) * sizeof(uint32_t));
  for (int64_t row = 0; row < n; row++) {
    int64_t row_base = row * k;
    for (int64_t g = 0; g < groups_per_row; g++) {
      double abs_max = 0;
      int64_t g_base = row_base + g * group_size;
      for (int64_t j = 0; j < group_size; j++) {
        double a = fabs((double)weight[g_base + j]);
        if (a > abs_max) abs_max = a;
      }
      /* f32ToF16Bits stores val into a Float32Array first: abs_max is already
       * an f32 value, so the (float) cast is exact. */
      uint16_t scale_bits = ref_f32_to_f16_bits((float)abs_max);
      scales[row * groups_per_row + g] = scale_bits;
      double scale = ref_f16_bits_to_f64(scale_bits);
      double inv = scale > 0 ? 127.0 / scale : 0.0;
      for (int64_t j = 0; j < group_size; j++) {
        double r = js_math_round((double)weight[g_base + j] * inv);
        /* Math.max(-127, Math.min(127, r)); NaN propagates, then NaN & 0xff = 0 */
        int32_t q;
        if (isnan(r)) q = 0;
        else if (r > 127.0) q = 127;
        else if (r < -127.0) q = -127;
        else q = (int32_t)r;
        int64_t k_idx = g * group_size + j;
        int64_t word = row * words_per_row + (k_idx >> 2);
        int byte = (int)(k_idx & 3);
        packed[word] |= ((uint32_t)q & 0xffu) << (byte * 8);
      }
    }
  }
  return 0;
}

/* ------------------------------------------------------------------ A3 */

/* src/backend/quantize.ts:138-156  dequantizeToF32:
 *   out = f32( (qi / 127) * f16->double(scale) ), qi a sign-extended byte,
 * -128 is NOT clamped. */
void ref_dequant_int8_grouped(const uint32_t* packed, const uint16_t* scales, int64_t n,
                              int64_t k, int64_t group_size, float* out) {
  int64_t groups_per_row = k / group_size;
  int64_t words_per_row = k / 4;
  for (int64_t row = 0; row < n; row++) {
    for (int64_t k_idx = 0; k_idx < k; k_idx++) {
      uint32_t word = packed[row * words_per_row + (k_idx >> 2)];
      int byte = (int)(k_idx & 3);
      int32_t qi = (int32_t)((word >> (byte * 8)) & 0xffu);
      if (qi >= 128) qi -= 256;
      int64_t g = k_idx / group_size;
      double scale = ref_f16_bits_to_f64(scales[row * groups_per_row + g]);
      out[row * k + k_idx] = (float)(((double)qi / 127.0) * scale);
    }
  }
}

/* int8 with one f32 scale per output row: w = f32(q * s).  The byte-lane
 * packing is the one of quantize.ts:121-125; the arithmetic is the benchmark
 * definition y = x.(W.s)^T.  q (8 bits) times s (24 bits) is exact in double,
 * so the single (float) cast is the correctly rounded product. */
void ref_dequant_int8_row(const uint32_t* packed, const float* row_scales, int64_t n, int64_t k,
                          float* out) {
  int64_t words_per_row = k / 4;
  for (int64_t row = 0; row < n; row++) {
    double s = (double)row_scales[row];
    for (int64_t k_idx = 0; k_idx < k; k_idx++) {
      uint32_t word = packed[row * words_per_row + (k_idx >> 2)];
      int32_t qi = (int32_t)((word >> ((k_idx & 3) * 8)) & 0xffu);
      if (qi >= 128) qi -= 256;
      out[row * k + k_idx] = (float)((double)qi * s);
    }
  }
}

/* int4 groupwise: docs/quantization-design.md:69-75 — 8 nibbles per u32 packed
 * 8-along-K into [N, K/8]; nibble j = (word >> 4j) & 0xF holds k = 8*word+j,
 * sign-extended from 4 bits; one f16 scale per group along K.  w = f32(q * s). */
void ref_dequant_int4_grouped(const uint32_t* packed, const uint16_t* scales, int64_t n, int64_t k,
                              int64_t group_size, float* out) {
  int64_t groups_per_row = k / group_size;
  int64_t words_per_row = k / 8;
  for (int64_t row = 0; row < n; row++) {
    for (int64_t k_idx = 0; k_idx < k; k_idx++) {
      uint32_t word = packed[row * words_per_row + (k_idx >> 3)];
      int32_t qi = (int32_t)((word >> ((k_idx & 7) * 4)) & 0xfu);
      if (qi >= 8) qi -= 16;
      double scale = ref_f16_bits_to_f64(scales[row * groups_per_row + k_idx / group_size]);
      out[row * k + k_idx] = (float)((double)qi * scale);
    }
  }
}

/* ----------------------------------------------------------------- A13 */

/* src/backend/cpu/numeric.ts:565-582  matmul inner loops, for the layout
 * api.linear produces (src/frontend/torchlette.ts:887-891): a is [M,K]
 * row-major, b is the transposed view of a row-major [N,K] weight.  acc is a
 * double; each product of two f32-valued doubles is exact; products are added
 * in increasing k; the Float32Array store rounds once.
 * threads <= 1 is the reference's single-threaded order of work; threads > 1
 * splits output columns over OpenMP threads (same arithmetic per element). */
void ref_matmul_nt(const float* a, const float* w, int64_t m, int64_t n, int64_t k, float* out,
                   int threads) {
#if defined(_OPENMP)
  if (threads > 1) {
#pragma omp parallel for num_threads(threads) schedule(static)
    for (int64_t col = 0; col < n; col++) {
      const float* wr = w + col * k;
      for (int64_t row = 0; row < m; row++) {
        const float* ar = a + row * k;
        double acc = 0;
        for (int64_t inner = 0; inner < k; inner++) acc += (double)ar[inner] * (double)wr[inner];
        out[row * n + col] = (float)acc;
      }
    }
    return;
  }
#endif
  (void)threads;
  for (int64_t row = 0; row < m; row++) {
    const float* ar = a + row * k;
    for (int64_t col = 0; col < n; col++) {
      const float* wr = w + col * k;
      double acc = 0;
      for (int64_t inner = 0; inner < k; inner++) acc += (double)ar[inner] * (double)wr[inner];
      out[row * n + col] = (float)acc;
    }
  }
}

/* General strided 2-D matmul, the same loop with explicit strides
 * (numeric.ts:553-582); used for the reference's own known answers. */
void ref_matmul_strided(const float* a, int64_t a_row_stride, int64_t a_inner_stride,
                        const float* b, int64_t b_inner_stride, int64_t b_col_stride, int64_t m,
                        int64_t n, int64_t k, float* out) {
  for (int64_t row = 0; row < m; row++) {
    for (int64_t col = 0; col < n; col++) {
      double acc = 0;
      for (int64_t inner = 0; inner < k; inner++) {
        acc += (double)a[row * a_row_stride + inner * a_inner_stride] *
               (double)b[inner * b_inner_stride + col * b_col_stride];
      }
      out[row * n + col] = (float)acc;
    }
  }
}

/* ------------------------------------------------------------ A10, A11 */

/* api.linear's bias add (torchlette.ts:892-894) on the CPU backend: a binary
 * add of f32 values in double, stored to f32; bias broadcasts over rows. */
void ref_bias_add(float* y, const float* bias, int64_t m, int64_t n) {
  for (int64_t r = 0; r < m; r++)
    for (int64_t c = 0; c < n; c++) y[r * n + c] = (float)((double)y[r * n + c] + (double)bias[c]);
}

/* src/ops/semantic/erf.ts:28-56  Abramowitz-Stegun 7.1.26, Horner order kept. */
static double erf_approx(double v) {
  double sign = v < 0 ? -1.0 : 1.0;
  double ax = fabs(v);
  double t = 1.0 / (1.0 + 0.3275911 * ax);
  double poly =
      ((((1.061405429 * t + -1.453152027) * t + 1.421413741) * t + -0.284496736) * t + 0.254829592) *
      t;
  return sign * (1.0 - poly * exp(-ax * ax));
}

enum { REF_UNARY_NONE = 0, REF_UNARY_RELU = 1, REF_UNARY_SILU = 2, REF_UNARY_GELU_TANH = 3,
       REF_UNARY_GELU_ERF = 4, REF_UNARY_SIGMOID = 5, REF_UNARY_TANH = 6 };

/* Unary ops as the CPU backend evaluates them (numeric.ts:439-446: double
 * body, one f32 store).  Term order follows the expression trees:
 *   relu  catalog.ts:104-109   where(x > 0, x, 0)
 *   silu  catalog.ts:88-93     x / (1 + exp(-x))
 *   sigmoid catalog.ts:81-86   1 / (1 + exp(-x))
 *   gelu (tanh) composite.ts:40-51
 *         (0.5*x) * (1 + tanh(0.7978845608 * (x + 0.044715 * (x*(x*x)))))
 *   gelu_erf  composite.ts:60-65  (0.5*x) * (1 + erf(x * SQRT1_2)) */
double ref_unary_scalar(int op, double x) {
  switch (op) {
    case REF_UNARY_RELU: return x > 0 ? x : 0.0;
    case REF_UNARY_SILU: return x / (1.0 + exp(-x));
    case REF_UNARY_SIGMOID: return 1.0 / (1.0 + exp(-x));
    case REF_UNARY_TANH: return tanh(x);
    case REF_UNARY_GELU_TANH:
      return (0.5 * x) * (1.0 + tanh(0.7978845608 * (x + 0.044715 * (x * (x * x)))));
    case REF_UNARY_GELU_ERF: return (0.5 * x) * (1.0 + erf_approx(x * 0.7071067811865476));
    default: return x;
  }
}

void ref_unary(int op, float* y, int64_t count) {
  for (int64_t i = 0; i < count; i++) y[i] = (float)ref_unary_scalar(op, (double)y[i]);
}

/* api.mul on the CPU backend: double product of two f32 values, one f32 store
 * (numeric.ts binary loop; the product of two f32 is exact in double, so this is
 * the IEEE f32 product). */
void ref_mul(const float* a, const float* b, float* out, int64_t count) {
  for (int64_t i = 0; i < count; i++) out[i] = (float)((double)a[i] * (double)b[i]);
}

/* rmsnorm(x, weight, eps) on the CPU backend, the decomposed forward of
 * src/frontend/decomposed-ops.ts:221-233: five ops, each storing f32.
 *   xSq    = mul(x, x)
 *   meanSq = mean(xSq, dim=-1)   numeric.ts:1022-1057: the running sum lives in a
 *            Float32Array cell, so every addition rounds to f32; then f32(sum / D)
 *   t      = add(meanSq, eps)    eps is a double
 *   inv    = rsqrt(t)            catalog.ts:96-97: 1 / sqrt(t)
 *   y      = mul(mul(x, inv), weight) */
void ref_rmsnorm(const float* x, const float* weight, float* y, int64_t m, int64_t d, double eps) {
  for (int64_t r = 0; r < m; r++) {
    const float* xr = x + r * d;
    float sum = 0.0f;
    for (int64_t i = 0; i < d; i++) {
      const float sq = (float)((double)xr[i] * (double)xr[i]);
      sum = (float)((double)sum + (double)sq);
    }
    const float mean = (float)((double)sum / (double)d);
    const float t = (float)((double)mean + eps);
    const float inv = (float)(1.0 / sqrt((double)t));
    for (int64_t i = 0; i < d; i++) {
      const float nrm = (float)((double)xr[i] * (double)inv);
      y[r * d + i] = (float)((double)nrm * (double)weight[i]);
    }
  }
}

int ref_max_threads(void) {
#if defined(_OPENMP)
  return omp_get_max_threads();
#else
  return 1;
#endif
}
