// Decode GEMV / skinny GEMM over packed weights with fused dequant, VALU form:
// the kernel and its launch templates.  The three weight formats are instantiated
// in three translation units (gemv_int4.hip, gemv_int8_grouped.hip,
// gemv_int8_row.hip) so that they compile in parallel; gemv.hip holds the host side.
// Stands in for the reference's gemvNTQuantI8 kernel
// (src/backend/webgpu/matmul/gemv.ts:365-466), which reads one u32 and one
// scale word per weight with scalar loads; here:
//
//  * weights stream from HBM as 16-byte chunks (32 int4 or 16 int8 weights per
//    lane per load), consecutive lanes on consecutive chunks of one row;
//  * a chunk is dequantised in registers to exact integer f16 pairs and dotted
//    against the activations with v_dot2_f32_f16 (f32 accumulate); the group
//    scale multiplies the chunk's partial sum, so no rounding happens before
//    the f32 accumulate;
//  * the activations x[M,K] are staged once per workgroup in LDS, laid out so
//    that lane-consecutive chunks read consecutive 16-byte units;
//  * a row is owned by `lpr` (16/32/64) lanes; their partial sums are combined
//    with DPP, and when `kw` waves split K the per-wave sums are combined
//    through LDS;
//  * workgroups walk over row blocks with a grid-sized stride, so a large N
//    (an LM head) reuses the staged activations.
//
// HBM-bound: algorithmic bytes per call are packed + scales + x + y.
#pragma once
#include "device_utils.h"
#include "gemv_args.h"

namespace tlhip {
namespace {



// dot of one 16-byte weight chunk with the matching x chunk held as NQ u32x4.
template <int FMT, typename XT>
struct ChunkDot;

template <>
struct ChunkDot<TLHIP_FMT_INT4_GROUPED, _Float16> {
  static constexpr int NQ = 4;
  half2_t q[16];
  __device__ __forceinline__ void unpack(const u32x4& w) {
    unpack_int4_word(w.x, q);
    unpack_int4_word(w.y, q + 4);
    unpack_int4_word(w.z, q + 8);
    unpack_int4_word(w.w, q + 12);
  }
  __device__ __forceinline__ float dot(const u32x4 (&xv)[NQ]) const {
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      d = __builtin_amdgcn_fdot2(q[4 * i + 0], as_half2(xv[i].x), d, false);
      d = __builtin_amdgcn_fdot2(q[4 * i + 1], as_half2(xv[i].y), d, false);
      d = __builtin_amdgcn_fdot2(q[4 * i + 2], as_half2(xv[i].z), d, false);
      d = __builtin_amdgcn_fdot2(q[4 * i + 3], as_half2(xv[i].w), d, false);
    }
    return d;
  }
};

template <int FMT>
struct ChunkDotInt8Half {
  static constexpr int NQ = 2;
  half2_t q[8];
  __device__ __forceinline__ void unpack(const u32x4& w) {
    unpack_int8_word(w.x, q);
    unpack_int8_word(w.y, q + 2);
    unpack_int8_word(w.z, q + 4);
    unpack_int8_word(w.w, q + 6);
  }
  __device__ __forceinline__ float dot(const u32x4 (&xv)[NQ]) const {
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      d = __builtin_amdgcn_fdot2(q[4 * i + 0], as_half2(xv[i].x), d, false);
      d = __builtin_amdgcn_fdot2(q[4 * i + 1], as_half2(xv[i].y), d, false);
      d = __builtin_amdgcn_fdot2(q[4 * i + 2], as_half2(xv[i].z), d, false);
      d = __builtin_amdgcn_fdot2(q[4 * i + 3], as_half2(xv[i].w), d, false);
    }
    return d;
  }
};
template <>
struct ChunkDot<TLHIP_FMT_INT8_GROUPED, _Float16> : ChunkDotInt8Half<TLHIP_FMT_INT8_GROUPED> {};
template <>
struct ChunkDot<TLHIP_FMT_INT8_ROW, _Float16> : ChunkDotInt8Half<TLHIP_FMT_INT8_ROW> {};

// f32 activations: weights become f32 integers, plain fma chain.
template <int FMT>
struct ChunkDotInt8Float {
  static constexpr int NQ = 4;
  float q[16];
  __device__ __forceinline__ void unpack(const u32x4& w) {
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      q[4 * i + 0] = (float)(int8_t)(words[i] & 0xffu);
      q[4 * i + 1] = (float)(int8_t)((words[i] >> 8) & 0xffu);
      q[4 * i + 2] = (float)(int8_t)((words[i] >> 16) & 0xffu);
      q[4 * i + 3] = (float)(int8_t)(words[i] >> 24);
    }
  }
  __device__ __forceinline__ float dot(const u32x4 (&xv)[NQ]) const {
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      d = fmaf(q[4 * i + 0], as_float(xv[i].x), d);
      d = fmaf(q[4 * i + 1], as_float(xv[i].y), d);
      d = fmaf(q[4 * i + 2], as_float(xv[i].z), d);
      d = fmaf(q[4 * i + 3], as_float(xv[i].w), d);
    }
    return d;
  }
};
template <>
struct ChunkDot<TLHIP_FMT_INT8_GROUPED, float> : ChunkDotInt8Float<TLHIP_FMT_INT8_GROUPED> {};
template <>
struct ChunkDot<TLHIP_FMT_INT8_ROW, float> : ChunkDotInt8Float<TLHIP_FMT_INT8_ROW> {};

template <>
struct ChunkDot<TLHIP_FMT_INT4_GROUPED, float> {
  static constexpr int NQ = 8;
  float q[32];
  __device__ __forceinline__ void unpack(const u32x4& w) {
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j) q[8 * i + j] = (float)(((int)(words[i] << (28 - 4 * j))) >> 28);
  }
  __device__ __forceinline__ float dot(const u32x4 (&xv)[NQ]) const {
    float d = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      d = fmaf(q[4 * i + 0], as_float(xv[i].x), d);
      d = fmaf(q[4 * i + 1], as_float(xv[i].y), d);
      d = fmaf(q[4 * i + 2], as_float(xv[i].z), d);
      d = fmaf(q[4 * i + 3], as_float(xv[i].w), d);
    }
    return d;
  }
};

// LDS layout of the staged activations: 16-byte unit (row m, quarter qd of
// chunk c) lives at unit index (m*NQ + qd)*nchunks + c, so the lanes of a row
// group, which hold consecutive c, read consecutive units.
//
// Work of one lane is a sequence of batches: U chunks x R rows of 16-byte
// weight loads (plus their scales).  The batches of all row blocks of the
// workgroup form one software pipeline: the loads of batch i+1 are issued
// before batch i is consumed, and the very first batch is issued right after
// the activation loads and before the LDS store and barrier, so HBM latency
// overlaps the staging, the arithmetic and the reductions.  The hot path has no
// per-lane branches: out-of-range chunks load a clamped address and contribute
// zero through their scale (or a select).
// `bid` / `nblk`: this workgroup's index among, and the number of, the workgroups
// that work on this problem (the whole grid for a single launch; a slice of it
// when several problems share one launch).
// MF4 (int4, f16 activations, MT = 4, R = 1): the dot products of up to four activation
// rows go through v_mfma_f32_4x4x4_16b_f16 instead of one v_dot2 chain per row.  The
// instruction multiplies 16 independent 4 x 4 blocks: in block b (lanes 4b .. 4b+3) lane
// 4b+i supplies row i of A (4 k-values of activation row i) and column i of B (the same 4
// k-values of ITS weight row), and receives column i of D = A * B in its four
// accumulators: D[m][i] = sum_k x[m][k] * w[row i][k] for m = 0..3.  So the four lanes of
// a block hold four different weight rows and the same 16-byte chunk; the unpacked chunk
// is consumed by 8 such instructions whatever M is, where the VALU form needs 16 dot2 per
// activation row.  Lane mapping: row in the quad = lane % 4, chunk slot = lane / 4 (16
// chunk slots per wave: "lanes per row" is 16).
template <int FMT, typename XT, int MT, int R, int U, bool MF4 = false>
__device__ __forceinline__ void gemv_body(const GemvArgs& a, const int bid, const int nblk) {
  static_assert(!MF4 || (FMT == TLHIP_FMT_INT4_GROUPED && sizeof(XT) == 2 && MT == 4 && R == 1),
                "the 4x4x4 form is built for int4 weights, f16 activations, four rows");
  using Dot = ChunkDot<FMT, XT>;
  constexpr int NQ = Dot::NQ;
  constexpr bool GROUPED = (FMT != TLHIP_FMT_INT8_ROW);
  extern __shared__ u32x4 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int kw_idx = wave & (a.kw - 1);
  const int rg = wave >> a.kw_shift;
  const int sub = MF4 ? (lane & 3) : (lane >> a.lpr_shift);
  const int lj = MF4 ? (lane >> 2) : (lane & (a.lpr - 1));
  const int cstride = a.lpr * a.kw;
  const int cfirst = kw_idx * a.lpr + lj;
  const int x_units_per_row = a.k * (int)sizeof(XT) / 16;  // 16-byte units per activation row
  const u32x4* xg = (const u32x4*)a.x;
  // MF4: the four lanes of a block read four different activation rows at the same
  // chunk; a skew of 16 units per row keeps them (and the 16 blocks) on 64 different
  // 16-byte units instead of 4 lanes on each bank.
  constexpr int XSKEW = MF4 ? 16 : 0;
  float* partial = (float*)(lds + (size_t)MT * NQ * a.nchunks + MT * XSKEW);  // kw x rows_per_wg x MT, if kw > 1
  const int row_in_wg = rg * a.rows_per_wave + sub * R;
  const int last_chunk = a.nchunks - 1;

  // Only raw loaded values live here: converting or selecting on a loaded value
  // at issue time would make the wave wait for the load it has just issued.
  struct Batch {
    u32x4 w[U][R];
    uint16_t s[U][R];  // f16 bits of the chunk's group scale
    float rs[R];       // int8-row: the row's scale
  };

  // Issue the loads of one batch: chunks cb + u*cstride (u < U) of R rows.
  auto load_batch = [&](Batch& b, int rb, int cb) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      // tail rows recompute the last row; their store is masked
      const int64_t row = min((int64_t)rb * a.rows_per_wg + row_in_wg + r, a.n - 1);
      const u32x4* wrow = a.packed + row * a.nchunks;
      const uint16_t* srow = (const uint16_t*)a.scales + row * a.groups_per_row;
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = cb + u * cstride;
        const int cc = min(c, last_chunk);
        b.w[u][r] = __builtin_nontemporal_load(wrow + cc);
        if (GROUPED) b.s[u][r] = srow[cc >> a.cpg_shift];
      }
      if (!GROUPED) b.rs[r] = ((const float*)a.scales)[row];  // every batch: no load under a branch
    }
  };

  float acc[R][MT];
  float row_scale[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    row_scale[r] = 1.f;
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;
  }

  auto compute_batch = [&](const Batch& b, int cb) {
    if constexpr (MF4) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = cb + u * cstride;
        const int cc = min(c, last_chunk);
        // this lane's operand row: activation row `sub` of the chunk (rows past M read the last one)
        const int xrow = min(sub, a.m - 1);
        u32x4 xq[NQ];
#pragma unroll
        for (int qd = 0; qd < NQ; ++qd) xq[qd] = lds[(xrow * NQ + qd) * a.nchunks + xrow * XSKEW + cc];
        Dot d;
        d.unpack(b.w[u][0]);
        float4_t dd = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int t = 0; t < 8; ++t) {
          // half2 pairs 2t, 2t+1 of the chunk, in the order the unpack produces (the
          // staged activations have the same order)
          const uint32_t xw[4] = {xq[t >> 1].x, xq[t >> 1].y, xq[t >> 1].z, xq[t >> 1].w};
          const half2_t x0 = as_half2(xw[(2 * t) & 3]), x1 = as_half2(xw[(2 * t + 1) & 3]);
          const half4_t av = {x0[0], x0[1], x1[0], x1[1]};
          const half2_t w0 = d.q[2 * t], w1 = d.q[2 * t + 1];
          const half4_t bv = {w0[0], w0[1], w1[0], w1[1]};
          dd = __builtin_amdgcn_mfma_f32_4x4x4f16(av, bv, dd, 0, 0, 0);
        }
        const float sc = c <= last_chunk ? half_bits_to_float(b.s[u][0]) : 0.f;
#pragma unroll
        for (int m = 0; m < 4; ++m) acc[0][m] = fmaf(sc, dd[m], acc[0][m]);
      }
      return;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = cb + u * cstride;
      const int cc = min(c, last_chunk);
      u32x4 xv[MT][NQ];
#pragma unroll
      for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int qd = 0; qd < NQ; ++qd) xv[m][qd] = lds[(m * NQ + qd) * a.nchunks + cc];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        Dot d;
        d.unpack(b.w[u][r]);
        const float sc = GROUPED ? (c <= last_chunk ? half_bits_to_float(b.s[u][r]) : 0.f) : 0.f;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          const float part = d.dot(xv[m]);
          if (GROUPED) acc[r][m] = fmaf(sc, part, acc[r][m]);
          else acc[r][m] += (c <= last_chunk ? part : 0.f);
        }
      }
    }
  };

  // Reduce, combine K-split partials, apply the epilogue and store one row block.
  auto finish = [&](int rb) {
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        if constexpr (MF4) {
          // the 16 lanes of a weight row are lane % 4 apart
          float v = acc[r][m];
          v += __shfl_xor(v, 4);
          v += __shfl_xor(v, 8);
          v += __shfl_xor(v, 16);
          v += __shfl_xor(v, 32);
          acc[r][m] = v;
        } else {
          acc[r][m] = group_sum(acc[r][m], a.lpr);
        }
      }

    if (a.kw > 1) {
      // split-K combine through LDS: partial[kw][row in wg][m]
      lds_barrier();
      if (lj == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < MT; ++m) partial[((kw_idx * a.rows_per_wg) + row_in_wg + r) * MT + m] = acc[r][m];
      }
      lds_barrier();
      if (kw_idx == 0 && lj == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            float s = 0.f;
            for (int w = 0; w < a.kw; ++w) s += partial[((w * a.rows_per_wg) + row_in_wg + r) * MT + m];
            acc[r][m] = s;
          }
      }
    }

    if (kw_idx == 0 && lj == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int64_t row = (int64_t)rb * a.rows_per_wg + row_in_wg + r;
        if (row < a.n) {
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            if (m < a.m) {
              float v = acc[r][m] * (row_scale[r] * a.scale_mul) * a.alpha;
              v = apply_epilogue(a.epi, v, row, (int64_t)m * a.n + row);
              store_out(a.y, a.y_dtype, (int64_t)m * a.n + row, v);
            }
          }
        }
      }
    }
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;
  };

  const int step_chunks = cstride * U;
  const int nsteps = a.nsteps;
  int rb = bid, step = 0;
  Batch cur;
  // Order of issue matters: loads return in order, so the (few) activation
  // loads go first, then the first weight batch; the LDS store then waits for
  // the activations only, and the barrier for LDS only.
  constexpr int XS = 4;  // activation units a thread holds while its weight loads are in flight
  const int units = a.nchunks * NQ;
  // MF4 stages the rows that exist (its lanes read row min(lane % 4, M - 1)); the dot2
  // form stages MT rows, the ones past M as copies of the last
  const int units_total = units * (MF4 ? a.m : MT);
  // idx -> (activation row m, 16-byte unit u) without a division: MT <= 4
  auto split = [&](int idx, int& m, int& u) {
    m = 0;
    u = idx;
#pragma unroll
    for (int i = 1; i < MT; ++i)
      if (u >= units) {
        u -= units;
        ++m;
      }
  };
  auto x_src = [&](int idx) {
    int m, u;
    split(idx, m, u);
    const int mm = m < a.m ? m : a.m - 1;  // rows beyond m replicate the last row; never stored
    return xg + (size_t)mm * x_units_per_row + u;
  };
  auto x_dst = [&](int idx) {
    int m, u;
    split(idx, m, u);
    const int c = u / NQ, qd = u - c * NQ;
    return lds + (m * NQ + qd) * a.nchunks + m * XSKEW + c;
  };
  if (a.pro.kind != TLHIP_PRO_NONE) {
    // What is staged is f(x): see stage_with_prologue.
    constexpr int E = 16 / (int)sizeof(XT);  // elements per 16-byte unit
    constexpr bool PERMUTE = FMT == TLHIP_FMT_INT4_GROUPED && sizeof(XT) == 2;
    const int T = (int)blockDim.x;
    auto unit_off = [&](int idx, int& m, int& u) {
      split(idx, m, u);
      const int mm = m < a.m ? m : a.m - 1;
      return (size_t)mm * x_units_per_row + u;
    };
    u32x4 xr[XS], orr[XS];
    if (a.pro.kind == TLHIP_PRO_GATED_MUL) {
      // f(x) = unary(gate) * up, elementwise: groups of XS units per thread; the
      // first weight batch is issued behind the first group's loads.
      const u32x4* ug = (const u32x4*)a.pro.operand;
      auto issue = [&](int base) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
          int m, u;
          const size_t off = unit_off(min(base + tid + i * T, units_total - 1), m, u);
          xr[i] = xg[off];
          orr[i] = ug[off];
        }
      };
      auto consume = [&](int base) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
          const int idx = base + tid + i * T;
          if (idx < units_total) {
            float g[E], up[E];
            unit_to_floats<XT>(xr[i], g);
            unit_to_floats<XT>(orr[i], up);
#pragma unroll
            for (int e = 0; e < E; ++e) g[e] = apply_unary(a.pro.unary, g[e]) * up[e];
            u32x4 v = floats_to_unit<XT>(g);
            if (PERMUTE) v = permute_x_for_int4(v);
            *x_dst(idx) = v;
          }
        }
      };
      issue(0);
      load_batch(cur, rb, cfirst);
      consume(0);
      for (int base = XS * T; base < units_total; base += XS * T) {
        issue(base);
        consume(base);
      }
    } else {
      // RMSNORM: pass 1 parks the raw rows in LDS (at their final places) and sums
      // the squares; after the workgroup-wide sum every thread rescales the units
      // it parked itself, so no barrier is needed between the passes beyond the
      // one of the sum.
      __shared__ float red[4][17];  // [m][wave], and [m][16] = 1 / rms of row m
      float ss[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) ss[m] = 0.f;
      auto issue = [&](int base) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
          int m, u;
          xr[i] = xg[unit_off(min(base + tid + i * T, units_total - 1), m, u)];
        }
      };
      auto park = [&](int base) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
          const int idx = base + tid + i * T;
          if (idx < units_total) {
            int m, u;
            split(idx, m, u);
            float f[E];
            unit_to_floats<XT>(xr[i], f);
            float sq = 0.f;
#pragma unroll
            for (int e = 0; e < E; ++e) sq = fmaf(f[e], f[e], sq);
#pragma unroll
            for (int mm = 0; mm < MT; ++mm) ss[mm] += (mm == m) ? sq : 0.f;
            *x_dst(idx) = xr[i];
          }
        }
      };
      // norm weights of a group's units (E floats each)
      const float* nw = (const float*)a.pro.operand;
      u32x4 wv[XS][E / 4];
      auto issue_w = [&](int base) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
          int m, u;
          split(min(base + tid + i * T, units_total - 1), m, u);
#pragma unroll
          for (int h = 0; h < E / 4; ++h) wv[i][h] = *(const u32x4*)(nw + (size_t)u * E + 4 * h);
        }
      };
      float inv[MT];
      auto rescale = [&](int base) {
#pragma unroll
        for (int i = 0; i < XS; ++i) {
          const int idx = base + tid + i * T;
          if (idx < units_total) {
            int m, u;
            split(idx, m, u);
            float f[E];
            unit_to_floats<XT>(*x_dst(idx), f);
            const float s = red[m][16];  // inv[m]: a register array indexed by m would live in scratch
#pragma unroll
            for (int h = 0; h < E / 4; ++h) {
              f[4 * h + 0] = (f[4 * h + 0] * s) * as_float(wv[i][h].x);
              f[4 * h + 1] = (f[4 * h + 1] * s) * as_float(wv[i][h].y);
              f[4 * h + 2] = (f[4 * h + 2] * s) * as_float(wv[i][h].z);
              f[4 * h + 3] = (f[4 * h + 3] * s) * as_float(wv[i][h].w);
            }
            u32x4 v = floats_to_unit<XT>(f);
            if (PERMUTE) v = permute_x_for_int4(v);
            *x_dst(idx) = v;
          }
        }
      };
      // the first group's rows and norm weights, then the first weight batch: the
      // sum below waits for the rows only
      issue(0);
      issue_w(0);
      load_batch(cur, rb, cfirst);
      park(0);
      for (int base = XS * T; base < units_total; base += XS * T) {
        issue(base);
        park(base);
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        ss[m] = group_sum(ss[m], 64);
        if (lane == 0) red[m][wave] = ss[m];
      }
      lds_barrier();
      const int nwaves = T >> 6;
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        float t = 0.f;
        for (int w = 0; w < nwaves; ++w) t += red[m][w];
        inv[m] = 1.f / sqrtf(t / (float)a.k + a.pro.eps);
      }
      // Every thread holds the same values and writes them all, so each reads back
      // what it wrote itself (a write by one lane for the others would need a barrier:
      // the compiler may move the other lanes' read ahead of it).
#pragma unroll
      for (int m = 0; m < MT; ++m) red[m][16] = inv[m];
      rescale(0);
      for (int base = XS * T; base < units_total; base += XS * T) {
        issue_w(base);
        rescale(base);
      }
    }
  } else
  if (units_total <= XS * (int)blockDim.x) {
    u32x4 xr[XS];
#pragma unroll
    for (int i = 0; i < XS; ++i) {
      const int idx = min(tid + i * (int)blockDim.x, units_total - 1);
      xr[i] = *x_src(idx);
    }
    load_batch(cur, rb, cfirst);
#pragma unroll
    for (int i = 0; i < XS; ++i) {
      // Unconditional store at the clamped place (a thread past the end writes again
      // what the last one writes): a store under a branch lets the compiler sink its
      // load into the branch, behind the weight loads, and wait there for all of them.
      const int idx = min(tid + i * (int)blockDim.x, units_total - 1);
      u32x4 v = xr[i];
      if (FMT == TLHIP_FMT_INT4_GROUPED && sizeof(XT) == 2) v = permute_x_for_int4(v);
      *x_dst(idx) = v;
    }
  } else {
    // groups of 8 units per thread: 8 loads in flight, then 8 LDS stores; the first
    // group's loads go ahead of the first weight batch (they come from L2 and return
    // first), the later groups queue behind it
    u32x4 xr[8];
    auto issue_x = [&](int base) {
#pragma unroll
      for (int i = 0; i < 8; ++i) xr[i] = *x_src(min(base + tid + i * (int)blockDim.x, units_total - 1));
    };
    auto store_x = [&](int base) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {  // unconditional, clamped: see above
        const int idx = min(base + tid + i * (int)blockDim.x, units_total - 1);
        u32x4 v = xr[i];
        if (FMT == TLHIP_FMT_INT4_GROUPED && sizeof(XT) == 2) v = permute_x_for_int4(v);
        *x_dst(idx) = v;
      }
    };
    issue_x(0);
    load_batch(cur, rb, cfirst);
    store_x(0);
    for (int base = 8 * (int)blockDim.x; base < units_total; base += 8 * (int)blockDim.x) {
      issue_x(base);
      store_x(base);
    }
  }
  lds_barrier();

  // Batches of this lane, in order: j -> (row block round j / nsteps, step j % nsteps).
  // Two register sets ping-pong with no copies between them, and every load inside
  // the steady-state loop is unconditional: a load under a branch makes the wait
  // counters at the join assume it was NOT issued, and the consumer of the other
  // set would then wait for the load just issued.
  const int rounds = (a.nblocks - bid + nblk - 1) / nblk;
  const int total = rounds * nsteps;
  auto advance = [&](int& r, int& st) {
    if (++st == nsteps) {
      st = 0;
      r += nblk;
    }
  };
  auto consume = [&](const Batch& b, int r, int st) {
    if (!GROUPED) {
#pragma unroll
      for (int i = 0; i < R; ++i) row_scale[i] = b.rs[i];
    }
    compute_batch(b, cfirst + st * step_chunks);
    if (st == nsteps - 1) finish(r);
  };
  Batch other;
  int j = 0;
  while (total - j >= 3) {
    int rb1 = rb, step1 = step;
    advance(rb1, step1);
    load_batch(other, rb1, cfirst + step1 * step_chunks);
    consume(cur, rb, step);
    rb = rb1;
    step = step1;
    advance(rb, step);
    load_batch(cur, rb, cfirst + step * step_chunks);
    consume(other, rb1, step1);
    j += 2;
  }
  if (total - j == 2) {
    int rb1 = rb, step1 = step;
    advance(rb1, step1);
    load_batch(other, rb1, cfirst + step1 * step_chunks);
    consume(cur, rb, step);
    consume(other, rb1, step1);
  } else if (total - j == 1) {
    consume(cur, rb, step);
  }
}

template <int FMT, typename XT, int MT, int R, int U, bool MF4 = false>
__global__ __launch_bounds__(512) void gemv_kernel(const GemvArgs a) {
  gemv_body<FMT, XT, MT, R, U, MF4>(a, blockIdx.x, gridDim.x);
}

// Several problems of one shape class (same format, K, activation type, rows and
// kernel configuration; N, pointers and epilogues differ) in ONE launch: a decode
// step issues q/k/v or gate/up on the same activations, each far too small to
// fill the chip, and every launch costs 2-3 us.  Workgroups
// [first[i], first[i+1]) work on problem i.

template <int FMT, typename XT, int MT, int R, int U>
__global__ __launch_bounds__(512) void gemv_grouped_kernel(const GroupedGemvArgs g) {
  int i = 0;
#pragma unroll
  for (int j = 1; j < kMaxGroup; ++j)
    if (j < g.count && (int)blockIdx.x >= g.first[j]) i = j;
  gemv_body<FMT, XT, MT, R, U>(g.p[i], (int)blockIdx.x - g.first[i], g.first[i + 1] - g.first[i]);
}

template <int FMT, typename XT, int MT, int R, int U, bool MF4 = false>
int launch_t(const GemvArgs& a, int threads, int grid, size_t lds_bytes, hipStream_t stream) {
  const void* fn = (const void*)gemv_kernel<FMT, XT, MT, R, U, MF4>;
  void* args[] = {(void*)&a};
  return launch_kernel(fn, dim3(grid), dim3(threads), args, lds_bytes, stream);
}

// (rows per lane group, chunks in flight) pairs that are instantiated: R*U <= 8.
template <int FMT, typename XT, int MT>
int launch_r(int r, int u, const GemvArgs& a, int threads, int grid, size_t lds_bytes, hipStream_t stream) {
  switch (r * 16 + u) {
    case 1 * 16 + 2: return launch_t<FMT, XT, MT, 1, 2>(a, threads, grid, lds_bytes, stream);
    case 1 * 16 + 4: return launch_t<FMT, XT, MT, 1, 4>(a, threads, grid, lds_bytes, stream);
    case 1 * 16 + 8: return launch_t<FMT, XT, MT, 1, 8>(a, threads, grid, lds_bytes, stream);
    case 2 * 16 + 2: return launch_t<FMT, XT, MT, 2, 2>(a, threads, grid, lds_bytes, stream);
    case 2 * 16 + 4: return launch_t<FMT, XT, MT, 2, 4>(a, threads, grid, lds_bytes, stream);
    case 4 * 16 + 2: return launch_t<FMT, XT, MT, 4, 2>(a, threads, grid, lds_bytes, stream);
  }
  return set_error(TLHIP_ERR_INVALID, "gemv: (rows per lane group, chunks in flight) = (%d,%d) is not built", r, u);
}

template <int FMT, typename XT>
int launch_m(int mt, int r, int u, const GemvArgs& a, int threads, int grid, size_t lds_bytes,
             hipStream_t stream) {
  switch (mt) {
    case 1: return launch_r<FMT, XT, 1>(r, u, a, threads, grid, lds_bytes, stream);
    case 2: return launch_r<FMT, XT, 2>(r, u, a, threads, grid, lds_bytes, stream);
    case 4: return launch_r<FMT, XT, 4>(r, u, a, threads, grid, lds_bytes, stream);
  }
  return set_error(TLHIP_ERR_INVALID, "gemv: internal M tile %d", mt);
}

template <int FMT>
int launch_x(int x_dtype, int mt, int r, int u, const GemvArgs& a, int threads, int grid, size_t lds_bytes,
             hipStream_t stream) {
  if (x_dtype == TLHIP_F16) return launch_m<FMT, _Float16>(mt, r, u, a, threads, grid, lds_bytes, stream);
  return launch_m<FMT, float>(mt, r, u, a, threads, grid, lds_bytes, stream);
}

template <int FMT, int R>
int launch_grouped_t(const GroupedGemvArgs& g, int threads, size_t lds_bytes, hipStream_t stream) {
  const void* fn = (const void*)gemv_grouped_kernel<FMT, _Float16, 1, R, 2>;
  void* args[] = {(void*)&g};
  return launch_kernel(fn, dim3(g.first[g.count]), dim3(threads), args, lds_bytes, stream);
}


}  // namespace

// One translation unit per weight format defines these two.
#define TLHIP_DEFINE_GEMV_FORMAT(NAME, FMT)                                                                   \
  int launch_gemv_##NAME(int x_dtype, int mt, int r, int u, const GemvArgs& a, int threads, int grid,          \
                         size_t lds_bytes, hipStream_t stream) {                                              \
    return launch_x<FMT>(x_dtype, mt, r, u, a, threads, grid, lds_bytes, stream);                             \
  }                                                                                                           \
  int launch_gemv_grouped_##NAME(int r, const GroupedGemvArgs& g, int threads, size_t lds_bytes,               \
                                 hipStream_t stream) {                                                        \
    return r == 1 ? launch_grouped_t<FMT, 1>(g, threads, lds_bytes, stream)                                   \
                  : launch_grouped_t<FMT, 2>(g, threads, lds_bytes, stream);                                  \
  }

}  // namespace tlhip
