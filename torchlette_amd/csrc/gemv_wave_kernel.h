// Skinny GEMM (1 <= M <= 16 activation rows) over int4 weights in groups of 32 on the
// matrix cores, built as one software pipeline PER WAVE over K: nothing is staged for the
// whole workgroup up front, and no workgroup barrier stands between a wave and its loads.
//
// Work split.  Weight rows go in blocks of 16; a workgroup owns RP row blocks (the launch
// has at most RP x workgroups of them) and its waves split K into W contiguous ranges of
// `steps` steps, a step being U 128-k iterations.  For a step a wave loads
//   * its own 128 U k of the activations, M rows x 256 U bytes, as whole rows (coalesced),
//   * for each row block the 16 x 64 U bytes of packed weights, in the MFMA B-operand
//     layout or (LINE, U = 2) as whole 128-byte lines, 8 rows to an instruction, that pass
//     through a wave-private LDS patch into the operand layout,
// D steps ahead of the one it computes (a ring of D register sets), so the activation
// loads of step t + D travel with the weight loads while step t feeds the matrix cores.
// The SCALES of a wave's whole K range (16 U bytes per row and step, contiguous per row)
// are loaded once, up front, as whole 16-byte pieces laid side by side, kept in the wave's
// LDS and read from there step by step: a load per step and row block of 8 or 16 bytes
// per row touches 16 cache lines for 128 or 256 useful bytes, and it is the number of
// lines a CU has in flight, not bytes, that its memory pipeline runs out of (measured:
// such loads cost a wave as much as the weight loads themselves).
// The activations pass through a wave-private LDS patch (written as loaded, read back in
// the A-operand layout; one wave's LDS accesses stay in order, so no barrier) and are
// used for every row block: each k of x is loaded once per workgroup, and the
// accumulators of all row blocks stay live across K.
// At the end the waves park their partial tiles in LDS, meet at ONE barrier, and all
// threads add the W partials of an output element in wave order, apply the epilogue and
// store.
//
// Every load of the steady state is unconditional and goes to a valid address: rows
// beyond M or N and steps beyond K are clamped to the start of their buffer (one line
// that every lane shares), and what they deliver is never used (a wave-uniform flag
// skips the arithmetic of a step beyond K; rows beyond N or M are never stored).  A load
// under a branch would make the wait counters at the join assume the worst, and a buffer
// load pushed out of range, although it moves no data, costs about 50 ns of the wave's
// time each (measured).  Buffer loads are used for their 32-bit offsets only.
//
// The arithmetic is that of gemv_mfma_kernel.h: weights enter v_mfma_f32_16x16x32_f16 as
// exact integers in f16, one MFMA covers one scale group, the group's scale multiplies
// the f32 result.
#pragma once
#include <cstddef>
#include <cstring>

#include "gemv_mfma_common.h"

namespace tlhip {

constexpr int kWaveScaleLoads = 6;  // 16-byte scale loads per lane at most (64 pieces each)

struct WaveArgs {
  const void* packed;
  const void* scales;
  const void* x;
  void* y;
  int n;
  int m;
  int kb;        // bytes of a packed weight row, K / 2
  int nsteps;    // steps of U iterations over all of K, K / (128 U)
  int steps;     // steps per wave: ceil(nsteps / waves)
  int spr;       // 16-byte scale pieces per row of a wave's K range: ceil(steps * 8 U / 16)
  int spr_recip; // ceil(65536 / spr)
  int nsl;       // scale loads per lane: ceil(RP * 16 * spr / 64)
  int wave_units;  // 16-byte LDS units of a wave's private region
  uint32_t packed_bytes, scales_bytes, x_bytes;
  float alpha;
  int y_dtype;
  DevEpilogue epi;
};

namespace {

__device__ __forceinline__ __amdgpu_buffer_rsrc_t wave_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// RP: row blocks per workgroup; MQ: 16-byte activation loads per lane and step (they cover
// MQ * 4 / U rows >= M); D: steps in flight; U: iterations per step; LINE: whole-line
// weight loads (U = 2).
template <int RP, int MQ, int D, int U, bool LINE>
__global__ __launch_bounds__(512) void gemv_wave_kernel(const WaveArgs a) {
  static_assert(!LINE || U == 2, "whole-line weight loads take two iterations per step");
  constexpr int RU = 16 * U + 1;  // units of a patch row: U iterations of 128 k + 1 pad
  constexpr int RPQ = 4 / U;      // activation rows per load instruction
  constexpr int WPATCH = LINE ? 128 : 0;
  extern __shared__ u32x4 lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = (int)(blockDim.x >> 6);
  const int nl = lane & 15;  // weight row inside a block (B operand), activation row (A operand)
  const int g = lane >> 4;   // k sub-block
  const int wg = blockIdx.x, nwg = gridDim.x;
  if (wg * 16 >= a.n) return;  // no row block is this workgroup's
  u32x4* patch = lds + wave * a.wave_units;  // activations of a step
  u32x4* wpatch = patch + 16 * RU;           // LINE: weights of a step and row block
  u32x4* sarea = wpatch + WPATCH;            // scales of the wave's K range: [row][spr pieces]
  float* parked = (float*)(lds + W * a.wave_units);  // [wave][RP][256]
  const __amdgpu_buffer_rsrc_t bw = wave_rsrc(a.packed, a.packed_bytes);
  const __amdgpu_buffer_rsrc_t bs = wave_rsrc(a.scales, a.scales_bytes);
  const __amdgpu_buffer_rsrc_t bx = wave_rsrc(a.x, a.x_bytes);
  const int st0 = wave * a.steps;  // first step of this wave's K range

  // ---- scales of the whole K range, first in the queue
  u32x4 sreg[kWaveScaleLoads];
#pragma unroll
  for (int i = 0; i < kWaveScaleLoads; ++i) {
    const int f = i * 64 + lane;
    const int ri = (f * a.spr_recip) >> 16;  // f / spr (exact for f < 384, spr <= 24)
    const int piece = f - ri * a.spr;
    const int row = ((ri >> 4) * nwg + wg) * 16 + (ri & 15);
    const int ok = (int)(i < a.nsl) & (int)(ri < RP * 16) & (int)(row < a.n);
    // A piece may reach past the wave's K range into the next row's scales (never read back),
    // and the last row's past the end of the buffer: a raw buffer load is range-checked dword
    // by dword, so what lies inside arrives and the rest reads as zero.
    const int off = (row * (a.kb >> 3) + st0 * (8 * U) + piece * 16) & -ok;
    sreg[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(bs, off, 0, 0));
  }

  u32x4 rw[D][RP][U];
  u32x4 rx[D][MQ];

  // This lane's place inside a step's activations (load q adds RPQ rows).
  const int xrow0 = lane / (16 * U);
  const int xunit = lane & (16 * U - 1);

  // The loads of this wave's step j into ring slot s.
  auto issue = [&](int s, int j) __attribute__((always_inline)) {
    const int st = st0 + j;
    const int mask = -(int)(st < a.nsteps);  // 0: a step beyond K, every offset becomes 0
#pragma unroll
    for (int q = 0; q < MQ; ++q) {
      const int row = min(RPQ * q + xrow0, a.m - 1);
      const int off = (row * (a.kb * 4) + st * (256 * U) + xunit * 16) & mask;
      rx[s][q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(bx, off, 0, 0));
    }
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      if constexpr (LINE) {
        // rows 0..7 of the block in register 0, rows 8..15 in register 1; lane = 8 * row + chunk
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int row = (r * nwg + wg) * 16 + 8 * h + (lane >> 3);
          const int rmask = mask & -(int)(row < a.n);
          rw[s][r][h] = __builtin_bit_cast(
              u32x4, __builtin_amdgcn_raw_buffer_load_b128(bw, (row * a.kb + st * 128 + (lane & 7) * 16) & rmask, 0, 2));
        }
      } else {
        const int row = (r * nwg + wg) * 16 + nl;
        const int rmask = mask & -(int)(row < a.n);
#pragma unroll
        for (int u = 0; u < U; ++u)
          rw[s][r][u] = __builtin_bit_cast(
              u32x4, __builtin_amdgcn_raw_buffer_load_b128(bw, (row * a.kb + (st * U + u) * 64 + g * 16) & rmask, 0, 2));
      }
    }
  };

  float4_t acc[RP];
#pragma unroll
  for (int r = 0; r < RP; ++r) acc[r] = (float4_t){0.f, 0.f, 0.f, 0.f};

  auto consume = [&](int s, int j) __attribute__((always_inline)) {
    if (st0 + j < a.nsteps) {  // wave-uniform: a step beyond K adds nothing
      // activations: into the wave's patch
#pragma unroll
      for (int q = 0; q < MQ; ++q) patch[(RPQ * q + xrow0) * RU + xunit] = permute_x_for_int4(rx[s][q]);
      // weights in the operand layout, and the step's 4 U scales of this lane's row
      u32x4 wv[RP][U];
      uint32_t sv[RP][2 * U];
#pragma unroll
      for (int r = 0; r < RP; ++r) {
        const char* at = (const char*)(sarea + (r * 16 + nl) * a.spr) + j * (8 * U);
        if constexpr (U == 1) {
          const uint2 v = *(const uint2*)at;
          sv[r][0] = v.x;
          sv[r][1] = v.y;
        } else {
          const u32x4 v = *(const u32x4*)at;
          sv[r][0] = v.x;
          sv[r][1] = v.y;
          sv[r][2] = v.z;
          sv[r][3] = v.w;
        }
        if constexpr (LINE) {
          const int r8 = lane >> 3, c8 = lane & 7;
          wpatch[r8 * 8 + (c8 ^ r8)] = rw[s][r][0];
          wpatch[(r8 + 8) * 8 + (c8 ^ r8)] = rw[s][r][1];
#pragma unroll
          for (int u = 0; u < U; ++u) wv[r][u] = wpatch[nl * 8 + ((g + 4 * u) ^ (nl & 7))];
        } else {
#pragma unroll
          for (int u = 0; u < U; ++u) wv[r][u] = rw[s][r][u];
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        half8_t xa[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) xa[t] = __builtin_bit_cast(half8_t, patch[nl * RU + 16 * u + 4 * t + g]);
#pragma unroll
        for (int r = 0; r < RP; ++r) {
          uint32_t w0 = wv[r][u].x, w1 = wv[r][u].y, w2 = wv[r][u].z, w3 = wv[r][u].w;
          transpose4(w0, w1, w2, w3);  // register t now holds word g of chunk 4*it + t
          const uint32_t ws[4] = {w0, w1, w2, w3};
          float4_t d[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            half2_t h[4];
            unpack_int4_word(ws[t], h);
            const float4_t zero = {0.f, 0.f, 0.f, 0.f};
            d[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t], join8(h), zero, 0, 0, 0);
          }
#pragma unroll
          for (int t = 0; t < 4; ++t) {
            const uint32_t wd = sv[r][2 * u + (t >> 1)];
            const float sc = half_bits_to_float((t & 1) ? (wd >> 16) : (wd & 0xffffu));
#pragma unroll
            for (int q = 0; q < 4; ++q) acc[r][q] = fmaf(sc, d[t][q], acc[r][q]);
          }
        }
      }
    }
  };

  // The loads of step j + D are issued behind the arithmetic of step j.  The steady-state
  // loop issues without conditions; the first D steps and the last 2D-1 at most are
  // handled around it.
  const int T = a.steps;
#pragma unroll
  for (int s = 0; s < D; ++s) {
    if (s < T) issue(s, s);
  }
  // the scales have arrived first: side by side into the wave's LDS
#pragma unroll
  for (int i = 0; i < kWaveScaleLoads; ++i) {
    if (i < a.nsl) sarea[i * 64 + lane] = sreg[i];
  }
  int t = 0;
  while (t + 2 * D <= T) {
#pragma unroll
    for (int s = 0; s < D; ++s) {
      consume(s, t + s);
      issue(s, t + s + D);
    }
    t += D;
  }
#pragma unroll
  for (int i = 0; i < 2 * D - 1; ++i) {
    if (t + i < T) {
      consume(i % D, t + i);
      if (t + i + D < T) issue(i % D, t + i + D);
    }
  }

  // ---- park, one barrier, all threads combine and store
#pragma unroll
  for (int r = 0; r < RP; ++r) {
#pragma unroll
    for (int q = 0; q < 4; ++q) parked[(wave * RP + r) * 256 + (4 * g + q) * 16 + nl] = acc[r][q];
  }
  lds_barrier();
  for (int o = tid; o < RP * 256; o += (int)blockDim.x) {
    const int r = o >> 8, e = o & 255;
    float sum = 0.f;
    for (int w = 0; w < W; ++w) sum += parked[(w * RP + r) * 256 + e];
    const int m = e >> 4;
    const int col = (r * nwg + wg) * 16 + (e & 15);
    if (col < a.n && m < a.m) {
      const int64_t idx = (int64_t)m * a.n + col;
      store_out(a.y, a.y_dtype, idx, apply_epilogue(a.epi, sum * a.alpha, col, idx));
    }
  }
}

}  // namespace
}  // namespace tlhip
