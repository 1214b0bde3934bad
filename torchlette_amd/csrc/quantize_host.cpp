// Host-side weight preparation: the f16 codec and the int8 group quantizer of
// src/backend/quantize.ts, as native code (the loader calls it once per
// projection tensor, examples/qwen3/loader.ts:231-252).  Rows are independent,
// so they are spread over host threads; each element is computed exactly as
// the reference does (double arithmetic, Math.round ties toward +infinity).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "common.h"

namespace {

inline uint32_t f32_bits(float v) {
  uint32_t u;
  std::memcpy(&u, &v, sizeof u);
  return u;
}

// quantize.ts:22-47.  Three regimes by the rebased exponent e16:
//   e16 >= 31      -> signed infinity pattern (also for NaN inputs)
//   1 <= e16 <= 30 -> normal: drop 13 mantissa bits, round to nearest even
//   e16 <= 0       -> subnormal: shift the 24-bit significand, add bit 12
//                     (ties go up), or signed zero below 2^-25
inline uint16_t encode_f16(float v) {
  const uint32_t u = f32_bits(v);
  const uint32_t sign = (u >> 16) & 0x8000u;
  const int e16 = int((u >> 23) & 0xffu) - 112;
  const uint32_t frac = u & 0x007fffffu;
  if (e16 >= 31) return uint16_t(sign | 0x7c00u);
  if (e16 >= 1) {
    uint32_t h = sign | (uint32_t(e16) << 10) | (frac >> 13);
    const uint32_t rem = frac & 0x1fffu;
    if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) h += 1;
    return uint16_t(h);
  }
  if (e16 < -10) return uint16_t(sign);
  const uint32_t shifted = (frac | 0x00800000u) >> uint32_t(1 - e16);
  return uint16_t(sign | ((shifted >> 13) + ((shifted >> 12) & 1u)));
}

// quantize.ts:50-60 (value is exact in double).
inline double decode_f16(uint16_t h) {
  const int e = (h >> 10) & 0x1f;
  const int f = h & 0x3ff;
  const double s = (h & 0x8000) ? -1.0 : 1.0;
  if (e == 0) return s * std::ldexp(double(f), -24);
  if (e == 31) return f ? std::nan("") : s * INFINITY;
  return s * std::ldexp(double(1024 + f), e - 25);
}

// ECMAScript Math.round for finite input: floor, then up if the fraction is
// at least one half (so -2.5 -> -2, 2.5 -> 3).
inline double round_half_up(double t) {
  const double f = std::floor(t);
  return (t - f >= 0.5) ? f + 1.0 : f;
}

void quantize_rows(const float* w, int64_t row_begin, int64_t row_end, int64_t k, int64_t g,
                   uint32_t* packed, uint16_t* scales) {
  const int64_t groups = k / g, words = k / 4;
  for (int64_t r = row_begin; r < row_end; ++r) {
    const float* wr = w + r * k;
    uint32_t* pr = packed + r * words;
    std::fill(pr, pr + words, 0u);
    for (int64_t gi = 0; gi < groups; ++gi) {
      const float* wg = wr + gi * g;
      float amax = 0.f;  // NaN never compares greater, as in the reference
      for (int64_t j = 0; j < g; ++j) {
        const float a = std::fabs(wg[j]);
        if (a > amax) amax = a;
      }
      const uint16_t sbits = encode_f16(amax);
      scales[r * groups + gi] = sbits;
      const double s = decode_f16(sbits);
      const double inv = s > 0 ? 127.0 / s : 0.0;
      for (int64_t j = 0; j < g; ++j) {
        const double t = double(wg[j]) * inv;
        int q = 0;  // NaN -> 0 (NaN & 0xff in JavaScript)
        if (t == t) {
          const double rr = std::isinf(t) ? t : round_half_up(t);
          q = rr > 127.0 ? 127 : (rr < -127.0 ? -127 : int(rr));
        }
        const int64_t kk = gi * g + j;
        pr[kk >> 2] |= (uint32_t(q) & 0xffu) << (8 * (kk & 3));
      }
    }
  }
}

}  // namespace

extern "C" {

uint16_t tlhip_f32_to_f16_bits(float value) { return encode_f16(value); }

float tlhip_f16_bits_to_f32(uint16_t bits) { return float(decode_f16(bits)); }

int tlhip_quantize_int8_grouped(const float* host_weight, int64_t n, int64_t k, int64_t group_size,
                                uint32_t* host_packed, uint16_t* host_scales) {
  if (!host_weight || !host_packed || !host_scales)
    return tlhip::set_error(TLHIP_ERR_INVALID, "quantize: null pointer");
  if (n < 0 || k < 0) return tlhip::set_error(TLHIP_ERR_INVALID, "quantize: negative shape");
  if (k % 4 != 0)
    return tlhip::set_error(TLHIP_ERR_INVALID, "quantize: K=%lld must be divisible by 4", (long long)k);
  if (group_size <= 0 || k % group_size != 0)
    return tlhip::set_error(TLHIP_ERR_INVALID, "quantize: K=%lld must be divisible by groupSize=%lld",
                            (long long)k, (long long)group_size);
  if (n == 0 || k == 0) return TLHIP_OK;
  unsigned hw = std::thread::hardware_concurrency();
  int64_t threads = std::max<int64_t>(1, std::min<int64_t>({(int64_t)(hw ? hw : 1), 16, n * k / (1 << 18)}));
  if (threads <= 1) {
    quantize_rows(host_weight, 0, n, k, group_size, host_packed, host_scales);
    return TLHIP_OK;
  }
  std::vector<std::thread> pool;
  const int64_t per = (n + threads - 1) / threads;
  for (int64_t t = 0; t < threads; ++t) {
    const int64_t b = t * per, e = std::min(n, b + per);
    if (b >= e) break;
    pool.emplace_back(quantize_rows, host_weight, b, e, k, group_size, host_packed, host_scales);
  }
  for (auto& th : pool) th.join();
  return TLHIP_OK;
}

}  // extern "C"
