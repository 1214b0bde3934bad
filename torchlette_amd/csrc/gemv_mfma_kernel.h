// Skinny GEMM (2 <= M <= 16 activation rows, and 17..64 rows as MT = 2 or 4 tiles of 16
// rows per weight row block) over packed weights on the matrix cores: the weights are
// streamed from HBM exactly once whatever M is.
//
// Weight rows are processed in blocks of 16.  A wave feeds v_mfma_f32_16x16x32_f16 with
//   A = activations  (lane l supplies x[m = l%16][8 k-values of sub-block l/16])
//   B = weights      (lane l supplies w[n = l%16][the same 8 k-values])
//   D = 16 m x 16 n  (lane l holds D[m = 4*(l/16)+r][n = l%16], r = 0..3)
// so every lane's four accumulators belong to ONE weight row n, and the
// per-group scale of that row is applied to the f32 result of each MFMA
// (acc += s * d).  The weights enter the MFMA as exact small integers in f16
// and the activations are f16 already, so every product is exact and nothing
// is rounded before the f32 accumulate.
//
// Weight loads are 16 bytes per lane.  For int4 (32 weights = one scale group
// per load) the four lanes that share a row exchange words with
// v_permlane32_swap / v_permlane16_swap (a 4x4 transpose), so that one MFMA
// covers exactly one scale group.  For int8 a 16-byte load is half an MFMA's K;
// the k-order inside an MFMA is free as long as the activations use the same
// order, so no exchange is needed.
//
// Activations (all of x, M*K f16, which must fit LDS) are staged row by row with
// a padded row stride, so the MFMA operand reads are free of bank conflicts.
// `kw` waves split K for one row block and combine their partial tiles through
// LDS; with kw = 1 a wave owns a row block alone and nothing is combined.  The
// weight loads of all row blocks of a workgroup form one software pipeline, as
// in the VALU kernel.
#pragma once
#include <cstring>

#include "gemv_mfma_common.h"

namespace tlhip {

// Up to four problems that share their activations (q/k/v, gate/up of a decode step) run
// as one launch: their 16-row blocks form one index space, a row block finds its problem
// through this table.
constexpr int kMfmaMaxGroup = 4;
struct MfmaProblem {
  const u32x4* packed;
  const void* scales;
  void* y;
  int64_t n;
  int first_block;  // index of this problem's first 16-row block in the launch's block space
  DevEpilogue epi;
};

struct MfmaArgs {
  MfmaProblem p[kMfmaMaxGroup];
  int count;
  const _Float16* x;
  float* workspace;   // split-K partial tiles: [(row block * ks + slice) * 256]
  int* counters;      // split-K arrival counters, one per row block; zero between launches
  int k;
  int m;
  int nchunks;        // 16-byte chunks per weight row
  int cpg_shift;      // log2(chunks per scale group), grouped formats
  int groups_per_row;
  int ks;             // K slices handled by different workgroups (1 = none, power of two)
  int ks_shift;
  int slice_iters;    // wave iterations (4 chunks each) per K slice (the shorter slices, if they differ)
  int slice_rem;      // iterations that do not divide over the slices: the first slice_rem slices take one more
  int iters;          // wave iterations over all of K
  int kw;             // waves that split a slice for one 16-row block (power of two)
  int kw_shift;
  int blocks_per_wg;  // 16-row blocks a workgroup works on at a time = waves / kw
  int nsteps;         // batches (U consecutive iterations each) per row block per wave
  int nblocks;        // 16-row blocks of all problems together
  int nwgblocks;      // ceil(nblocks / blocks_per_wg)
  float alpha;
  float scale_mul;
  int y_dtype;
  int patch_unit;     // whole-line form: first 16-byte LDS unit of the waves' patches
};

namespace {

template <int FMT>
struct MfmaTraits;
template <>
struct MfmaTraits<TLHIP_FMT_INT4_GROUPED> {
  static constexpr int STEPS = 4;        // MFMAs per iteration (4 chunks x 32 weights)
};
template <>
struct MfmaTraits<TLHIP_FMT_INT8_GROUPED> {
  static constexpr int STEPS = 2;        // 4 chunks x 16 weights = 64 k
};
template <>
struct MfmaTraits<TLHIP_FMT_INT8_ROW> {
  static constexpr int STEPS = 2;
};

// Activations live in LDS row by row, as in global memory, 16-byte units, each
// row padded by one unit: the 16 lanes of an MFMA operand read (16 different
// rows, same k) then fall in 16 different bank groups, and staging is a
// straight coalesced copy.  The unit of row m that holds the 8 k-values of MFMA
// step t (counted over all of K), k sub-block g:
//   int4: k = 32*t + 8*g             -> unit 4*t + g
//   int8: k = 64*(t/2) + 16*g + 8*(t%2) -> unit 8*(t/2) + 2*g + (t%2)
template <int FMT>
__device__ __forceinline__ int x_unit(int t, int g, int m, int row_units) {
  const int ku = FMT == TLHIP_FMT_INT4_GROUPED ? 4 * t + g : 8 * (t >> 1) + 2 * g + (t & 1);
  return m * row_units + ku;
}

//
// LINE (U even; built for both int8 formats and for int4 with group size 32): a wave's
// weight loads take whole 128-byte lines, 8 lanes to a row and 8 rows to an instruction,
// with the nontemporal hint, instead of the operand layout's 64-byte pieces of 16 rows; a batch
// then goes through a wave-private LDS patch (written as loaded, read back in the
// operand layout, no barrier: one wave's LDS accesses stay in order) before it is
// consumed exactly as before.  A read-only kernel streams the LM head's 590 MB in
// 84-86 us with the first load shape and in 94-95 us (plain) or 102-106 us (hint) with
// the second.
//
// MT (1, 2, 4): tiles of 16 activation rows per weight row block.  A dequantised weight
// operand feeds MT MFMAs, one per tile, and everything that holds a 16 x 16 result
// (accumulators, parked tiles, K-slice tiles in the workspace) holds MT of them.
template <int FMT, int U, bool WIDE, int MAXT, bool LINE, bool GROUP, int MT = 1>
__global__ __launch_bounds__(MAXT) void gemv_mfma_kernel(const MfmaArgs a) {
  static_assert(!LINE || U % 2 == 0, "whole-line loads: an even number of iterations in flight");
  using Tr = MfmaTraits<FMT>;
  constexpr int STEPS = Tr::STEPS;
  constexpr bool GROUPED = (FMT != TLHIP_FMT_INT8_ROW);
  extern __shared__ u32x4 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int kw_idx = wave & (a.kw - 1);  // which K part of the row block
  const int bw_idx = wave >> a.kw_shift; // which row block of the workgroup
  const int nl = lane & 15;   // weight row inside the block / activation row for the A operand
  const int g = lane >> 4;    // k sub-block
  const int mrows = a.m;
  int ml[MT];  // this lane's activation row in each tile; rows beyond M alias the last row, never stored
#pragma unroll
  for (int t = 0; t < MT; ++t) ml[t] = min(16 * t + nl, mrows - 1);

  // A workgroup keeps ONE K slice (all of K when ks == 1) of the activations in
  // LDS and walks row-block groups with a grid stride; the ks workgroups of
  // consecutive blockIdx take the ks slices of the same row-block groups.
  const int slice = blockIdx.x & (a.ks - 1);
  const int wg_stride = gridDim.x >> a.ks_shift;
  int wgb = blockIdx.x >> a.ks_shift;
  // K slices of unequal length (K = 11008: 86 iterations over 4 slices = 22, 22, 21, 21)
  int my_iters = a.slice_iters, it_begin = slice * a.slice_iters, nsteps = a.nsteps;
  if (a.slice_rem) {
    my_iters += slice < a.slice_rem ? 1 : 0;
    it_begin += min(slice, a.slice_rem);
    nsteps = (my_iters / U + a.kw - 1) >> a.kw_shift;
  }
  constexpr int UNITS_PER_ITER = FMT == TLHIP_FMT_INT4_GROUPED ? 16 : 8;  // 16-byte x units per iteration
  const int slice_units = my_iters * UNITS_PER_ITER;  // resident x units per row
  const int row_units = slice_units + 1;                    // padded LDS row stride
  const int ku0 = it_begin * UNITS_PER_ITER;                // first resident unit
  const int k_units = a.k >> 3;                             // units per activation row in memory
  float* partial = (float*)(lds + (size_t)row_units * mrows);

  // A wave's batch = U consecutive iterations; batch `kw_idx + step * kw` of the
  // slice.  Raw loaded values only (no conversion at issue time, see gemv.hip).
  // Scales: a separate 2-byte load per MFMA step made the kernel 2.5x slower
  // than the weight stream alone (five memory instructions per kilobyte of
  // weights), so with one scale per 32 weights (WIDE) the 4*U scales of a
  // batch, contiguous in memory, come as U 8-byte or U/2 16-byte loads.
  constexpr int NS = FMT == TLHIP_FMT_INT4_GROUPED ? 4 : 1;  // distinct scales per iteration at most
  struct Batch {
    u32x4 w[U];
    uint16_t s[U][NS];      // !WIDE
    uint32_t sv[2 * U];     // WIDE: scale 4u+s in half (s & 1) of word 2u + s/2
  };
  const int nbatches = my_iters / U;  // U divides the iterations of a slice

  // row block of the launch -> its problem (wave-uniform).  In the hot loop the problem's
  // fields are SELECTED from the four table entries, each read with a constant index (so
  // they sit in scalar registers from the start of the kernel): indexing the kernel
  // arguments with a run-time index puts scalar loads, and their waits, which are also
  // waits for the LDS reads in flight, into every batch (measured: 1-3 us per launch).
  auto problem_of = [&](int rb) {
    int pi = 0;
    if constexpr (GROUP) {
#pragma unroll
      for (int j = 1; j < kMfmaMaxGroup; ++j)
        if (j < a.count && rb >= a.p[j].first_block) pi = j;
    }
    return pi;
  };
  struct Where {
    const u32x4* packed;
    const void* scales;
    int64_t n;
    int first_block;
  };
  auto locate = [&](int rb) {
    Where w{a.p[0].packed, a.p[0].scales, a.p[0].n, 0};
    if constexpr (GROUP) {
#pragma unroll
    for (int j = 1; j < kMfmaMaxGroup; ++j) {
      const bool here = j < a.count && rb >= a.p[j].first_block;
      w.packed = here ? a.p[j].packed : w.packed;
      w.scales = here ? a.p[j].scales : w.scales;
      w.n = here ? a.p[j].n : w.n;
      w.first_block = here ? a.p[j].first_block : w.first_block;
    }
    }
    return w;
  };

  auto load_batch = [&](Batch& b, int wb, int step) {
    const int rb = min(wb * a.blocks_per_wg + bw_idx, a.nblocks - 1);
    const Where P = locate(rb);
    const int64_t r0 = (int64_t)(rb - P.first_block) * 16;  // first row of the block inside its problem
    const int64_t row = min(r0 + nl, P.n - 1);
    const u32x4* wrow = P.packed + row * a.nchunks;
    const uint16_t* srow = (const uint16_t*)P.scales + row * a.groups_per_row;
    const int itb = it_begin + min(kw_idx + step * a.kw, nbatches - 1) * U;
    if constexpr (LINE) {
      // pair p of the batch = 128 k = one line per row: rows 0..7 of the block in
      // register 2p, rows 8..15 in register 2p+1, lane = 8 * row + 16-byte chunk
      const int r8 = lane >> 3, c8 = lane & 7;
      const int64_t row_lo = min(r0 + r8, P.n - 1);
      const int64_t row_hi = min(r0 + 8 + r8, P.n - 1);
      const u32x4* wlo = P.packed + row_lo * a.nchunks + c8;
      const u32x4* whi = P.packed + row_hi * a.nchunks + c8;
#pragma unroll
      for (int p2 = 0; p2 < U / 2; ++p2) {
        b.w[2 * p2] = __builtin_nontemporal_load(wlo + (itb + 2 * p2) * 4);
        b.w[2 * p2 + 1] = __builtin_nontemporal_load(whi + (itb + 2 * p2) * 4);
      }
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        // Nontemporal loads for the grouped formats (measured 0.3-0.5 us per call faster at
        // the 8-28 MB decode shapes); plain loads for one scale per row, the format of the
        // 590 MB LM head, where they measured 5 % faster (115.7 -> 110.1 us at M = 8).
        if (GROUPED) b.w[u] = __builtin_nontemporal_load(wrow + (itb + u) * 4 + g);
        else b.w[u] = wrow[(itb + u) * 4 + g];
      }
    }
    if (WIDE && FMT == TLHIP_FMT_INT8_GROUPED) {
      // group size 64 = one scale per iteration: the U scales of a batch, contiguous and
      // aligned (U divides the iterations of a row), as one 4- or 8-byte load
      static_assert(!(WIDE && FMT == TLHIP_FMT_INT8_GROUPED) || U == 2 || U == 4, "wide int8 scales: U = 2 or 4");
      if (U == 2) {
        b.sv[0] = *(const uint32_t*)(srow + itb);
      } else {
        const uint2 v = *(const uint2*)(srow + itb);
        b.sv[0] = v.x;
        b.sv[1] = v.y;
      }
    } else if (WIDE) {
      if (U == 1) {
        const uint2 v = *(const uint2*)(srow + itb * 4);
        b.sv[0] = v.x;
        b.sv[1] = v.y;
      } else {
#pragma unroll
        for (int h = 0; h < U / 2; ++h) {
          const u32x4 v = *(const u32x4*)(srow + itb * 4 + h * 8);  // 16-byte aligned: K % 256 == 0
          b.sv[4 * h + 0] = v.x;
          b.sv[4 * h + 1] = v.y;
          b.sv[4 * h + 2] = v.z;
          b.sv[4 * h + 3] = v.w;
        }
      }
    } else if (GROUPED) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int s = 0; s < NS; ++s) b.s[u][s] = srow[((itb + u) * 4 + s) >> a.cpg_shift];
      }
    }
  };

  float4_t acc[MT];
  // one scale per row (no per-group f32 step between the MFMAs): two accumulators take
  // the MFMA steps in turn, so that consecutive MFMAs of a wave do not depend on each other
  float4_t acc_odd[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    acc[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
    acc_odd[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
  }

  auto compute_batch = [&](const Batch& b, int step) __attribute__((always_inline)) {
    const int bidx = kw_idx + step * a.kw;
    const bool valid = bidx < nbatches;  // wave-uniform
    const int tlb = min(bidx, nbatches - 1) * U * STEPS;
    u32x4 wv[U];
    if constexpr (LINE) {
      // through the wave's patch: 16 rows x 8 chunks per pair, the chunk position
      // XOR-ed with the row so that the operand reads (16 rows, one chunk) spread
      // over the banks
      u32x4* st = lds + a.patch_unit + wave * (U / 2 * 128);
      const int r8 = lane >> 3, c8 = lane & 7;
#pragma unroll
      for (int p2 = 0; p2 < U / 2; ++p2) {
        st[p2 * 128 + r8 * 8 + (c8 ^ r8)] = b.w[2 * p2];
        st[p2 * 128 + (r8 + 8) * 8 + (c8 ^ r8)] = b.w[2 * p2 + 1];
      }
#pragma unroll
      for (int u = 0; u < U; ++u)
        wv[u] = st[(u >> 1) * 128 + nl * 8 + ((g + 4 * (u & 1)) ^ (nl & 7))];
    } else {
#pragma unroll
      for (int u = 0; u < U; ++u) wv[u] = b.w[u];
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int tl = tlb + u * STEPS;
      uint32_t w0 = wv[u].x, w1 = wv[u].y, w2 = wv[u].z, w3 = wv[u].w;
      half8_t bw[STEPS];
      if (FMT == TLHIP_FMT_INT4_GROUPED) {
        transpose4(w0, w1, w2, w3);  // register s now holds word g of chunk 4*it+s
        const uint32_t ws[4] = {w0, w1, w2, w3};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          half2_t h[4];
          unpack_int4_word(ws[s], h);
          bw[s] = join8(h);
        }
      } else {
        const uint32_t ws[4] = {w0, w1, w2, w3};
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          half2_t h[4];
          unpack_int8_word(ws[2 * s], h);
          unpack_int8_word(ws[2 * s + 1], h + 2);
          bw[s] = join8(h);
        }
      }
      if (!GROUPED) {
        // one scale per row, applied at the end: accumulate in the matrix core
        if (valid) {
#pragma unroll
          for (int s = 0; s < STEPS; ++s) {
#pragma unroll
            for (int t = 0; t < MT; ++t) {
              const u32x4 xa = lds[x_unit<FMT>(tl + s, g, ml[t], row_units)];
              if (s & 1) acc_odd[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xa), bw[s], acc_odd[t], 0, 0, 0);
              else acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xa), bw[s], acc[t], 0, 0, 0);
            }
          }
        }
      } else if (FMT == TLHIP_FMT_INT8_GROUPED) {
        // both steps of an iteration lie in one scale group
        const uint16_t sbits = WIDE ? (uint16_t)((u & 1) ? (b.sv[u >> 1] >> 16) : (b.sv[u >> 1] & 0xffffu)) : b.s[u][0];
        const float sc = valid ? half_bits_to_float(sbits) : 0.f;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const u32x4 xa0 = lds[x_unit<FMT>(tl, g, ml[t], row_units)];
          const u32x4 xa1 = lds[x_unit<FMT>(tl + 1, g, ml[t], row_units)];
          float4_t d = {0.f, 0.f, 0.f, 0.f};
          d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xa0), bw[0], d, 0, 0, 0);
          d = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xa1), bw[1], d, 0, 0, 0);
#pragma unroll
          for (int r = 0; r < 4; ++r) acc[t][r] = fmaf(sc, d[r], acc[t][r]);
        }
      } else {
        float sc[STEPS];
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
          uint16_t bits;
          if (WIDE) {
            const uint32_t wd = b.sv[2 * u + (s >> 1)];
            bits = (uint16_t)((s & 1) ? (wd >> 16) : (wd & 0xffffu));
          } else {
            bits = b.s[u][s];
          }
          sc[s] = valid ? half_bits_to_float(bits) : 0.f;
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          float4_t d[STEPS];
#pragma unroll
          for (int s = 0; s < STEPS; ++s) {
            const u32x4 xa = lds[x_unit<FMT>(tl + s, g, ml[t], row_units)];
            const float4_t zero = {0.f, 0.f, 0.f, 0.f};
            d[s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, xa), bw[s], zero, 0, 0, 0);
          }
#pragma unroll
          for (int s = 0; s < STEPS; ++s) {
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[t][r] = fmaf(sc[s], d[s][r], acc[t][r]);
          }
        }
      }
    }
  };

  // The finished 16 x 16 tiles of one row block (all of this workgroup's K), one per tile
  // of activation rows: combine with the other workgroups' K slices when ks > 1, apply the
  // epilogue, store.
  auto emit = [&](int rb, float4_t (&tile)[MT]) __attribute__((always_inline)) {
    bool owner = true;  // wave-uniform
    if (a.ks > 1) {
      // Publish this slice's tiles; the workgroup that arrives last for the row
      // block adds the ks tiles in slice order (so the sum does not depend on
      // who is last), resets the counter for the next launch and stores.
      // Tiles and counters move with device-scope atomic accesses only: those
      // are coherent between the L2 caches of the chip by themselves, and a
      // device-scope fence (a write-back and invalidate of a whole L2 per row
      // block) measured 3x slower for the whole kernel.  Order: tile stores,
      // wait until the memory system has acknowledged them, then the counter.
      // Every access to tiles and counters here and in sum_slices must stay a
      // device-scope atomic: a plain load could be served from this XCD's L2.
      float* mine = a.workspace + ((size_t)rb * a.ks + slice) * (MT * 256);
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          __hip_atomic_store(mine + t * 256 + (4 * g + r) * 16 + nl, tile[t][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): every store of this wave is acknowledged
      int old = 0;
      if (lane == 0) old = __hip_atomic_fetch_add(a.counters + rb, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      old = __shfl(old, 0);
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      owner = old == a.ks - 1;
      if (owner) {
        const float* tiles = a.workspace + (size_t)rb * a.ks * (MT * 256);
#pragma unroll
        for (int t = 0; t < MT; ++t) tile[t] = sum_slices(tiles + t * 256, a.ks, (4 * g) * 16 + nl, MT * 256);
        if (lane == 0) __hip_atomic_store(a.counters + rb, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (owner) {
      const MfmaProblem& P = a.p[problem_of(rb)];
      const int64_t orow = (int64_t)(rb - P.first_block) * 16 + nl;
      if (orow < P.n) {
        float rs = a.scale_mul * a.alpha;
        if (!GROUPED) rs *= ((const float*)P.scales)[orow];
        if constexpr (MT == 1) {
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const int m = 4 * g + r;
            if (m < mrows) {
              const float v = apply_epilogue(P.epi, tile[0][r] * rs, orow, (int64_t)m * P.n + orow);
              store_out(P.y, a.y_dtype, (int64_t)m * P.n + orow, v);
            }
          }
        } else {
          float v[MT * 4];
#pragma unroll
          for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) v[4 * t + r] = tile[t][r] * rs;
          apply_epilogue_all(P.epi, v, orow, [&](int j) -> int64_t {
            const int m = 16 * (j >> 2) + 4 * g + (j & 3);
            return m < mrows ? (int64_t)m * P.n + orow : (int64_t)-1;
          });
#pragma unroll
          for (int t = 0; t < MT; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int m = 16 * t + 4 * g + r;
              if (m < mrows) store_out(P.y, a.y_dtype, (int64_t)m * P.n + orow, v[4 * t + r]);
            }
        }
      }
    }
  };

  // End of a row block for this wave.  kw == 1: the wave owns the block, emit it.
  // kw > 1: park the wave's partial tile in LDS slot (round, wave) and go on; the
  // kw tiles of every block are combined after the main loop, behind ONE barrier.
  // (A combine per row block cost two barriers, i.e. two waits for the slowest
  // wave's memory latency, and with K slices one drain of the load pipeline, per
  // block: 3 us of a 12 us kernel, 6 us with four K slices.)
  int round = 0;
  auto finish = [&](int wb) __attribute__((always_inline)) {
    if (!GROUPED) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        acc[t] += acc_odd[t];
        acc_odd[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
      }
    }
    if (a.kw == 1) {
      const int rb = wb * a.blocks_per_wg + bw_idx;
      if (rb < a.nblocks) emit(rb, acc);
    } else {
      float* tile = partial + (size_t)(round * (int)(blockDim.x >> 6) + wave) * (MT * 256);
#pragma unroll
      for (int t = 0; t < MT; ++t)
#pragma unroll
        for (int r = 0; r < 4; ++r) tile[t * 256 + (4 * g + r) * 16 + nl] = acc[t][r];
    }
    ++round;
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
  };

  // Activations first (they return first), then the first weight batch, then
  // the LDS store; consecutive threads on consecutive 16-byte units of a row.
  const u32x4* xg = (const u32x4*)a.x + ku0;
  const int res_units = slice_units;
  int step = 0;
  Batch cur;
  if (res_units <= (int)blockDim.x && mrows <= 4) {
    u32x4 xr[4];
    const int ku = min(tid, res_units - 1);
#pragma unroll
    for (int m = 0; m < 4; ++m) xr[m] = xg[(size_t)min(m, mrows - 1) * k_units + ku];
    load_batch(cur, wgb, 0);
    // Unconditional stores at clamped places (a thread past the end, or a row past
    // M, writes again what its neighbour writes): a store under a branch lets the
    // compiler sink its load into the branch, behind the weight loads, and wait there
    // for everything in flight (0.2-0.9 us per launch).
#pragma unroll
    for (int m = 0; m < 4; ++m) {
      u32x4 v = xr[m];
      if (FMT == TLHIP_FMT_INT4_GROUPED) v = permute_x_for_int4(v);
      lds[min(m, mrows - 1) * row_units + ku] = v;
    }
  } else {
    // The mrows x res_units resident units as one flat index, consecutive threads on
    // consecutive units of a row; a thread issues a group of 16 loads, then the first
    // weight batch, then stores the group to LDS.  The copy is bound by the latency of
    // a round trip to L2, so what counts is the number of rounds (16 rows of K = 4096,
    // or of a 3072-wide slice, on 512 threads: one).  A place past the end loads
    // nothing and stores to the padding unit of the last row, which nobody reads: the
    // store stays unconditional (see above), the load is what costs.
    constexpr int G = 16;
    const int T = (int)blockDim.x;
    const int total_units = mrows * res_units;
    const int pad = (mrows - 1) * row_units + res_units;
    // idx -> (row, unit): one division per thread, then stepped by T
    const int qT = T / res_units, rT = T - qT * res_units;
    int m = tid / res_units, ku = tid - m * res_units;
    u32x4 xr[G];
    int dst[G];
    auto issue_x = [&]() {
#pragma unroll
      for (int i = 0; i < G; ++i) {
        xr[i] = (u32x4){0u, 0u, 0u, 0u};
        dst[i] = pad;
        if (m < mrows) {
          xr[i] = xg[(size_t)m * k_units + ku];
          dst[i] = m * row_units + ku;
        }
        m += qT;
        ku += rT;
        if (ku >= res_units) {
          ku -= res_units;
          ++m;
        }
      }
    };
    auto store_x = [&]() {
#pragma unroll
      for (int i = 0; i < G; ++i) {
        u32x4 v = xr[i];
        if (FMT == TLHIP_FMT_INT4_GROUPED) v = permute_x_for_int4(v);
        lds[dst[i]] = v;
      }
    };
    issue_x();
    load_batch(cur, wgb, 0);
    store_x();
    for (int base = G * T; base < total_units; base += G * T) {
      issue_x();
      store_x();
    }
  }
  lds_barrier();

  // Batches of this wave, in order: j -> (workgroup round j / nsteps, step j % nsteps).
  // Two register sets ping-pong with no copies between them, and every load inside
  // the steady-state loop is unconditional: a load under a branch makes the wait
  // counters at the join assume it was NOT issued, and the consumer of the other
  // set would then wait for the load just issued.
  const int rounds = (a.nwgblocks - wgb + wg_stride - 1) / wg_stride;
  const int total = rounds * nsteps;
  auto advance = [&](int& b, int& st) {
    if (++st == nsteps) {
      st = 0;
      b += wg_stride;
    }
  };
  auto consume = [&](const Batch& b, int wb, int st) __attribute__((always_inline)) {
    compute_batch(b, st);
    if (st == nsteps - 1) finish(wb);
  };
  Batch other;
  int j = 0;
  while (total - j >= 3) {
    int wgb1 = wgb, step1 = step;
    advance(wgb1, step1);
    load_batch(other, wgb1, step1);
    consume(cur, wgb, step);
    wgb = wgb1;
    step = step1;
    advance(wgb, step);
    load_batch(cur, wgb, step);
    consume(other, wgb1, step1);
    j += 2;
  }
  if (total - j == 2) {
    int wgb1 = wgb, step1 = step;
    advance(wgb1, step1);
    load_batch(other, wgb1, step1);
    consume(cur, wgb, step);
    consume(other, wgb1, step1);
  } else if (total - j == 1) {
    consume(cur, wgb, step);
  }

  if (a.kw > 1) {
    // the parked tiles: rounds x blocks_per_wg of them, dealt to the waves
    lds_barrier();
    const int waves = (int)(blockDim.x >> 6);
    const int bshift = __builtin_ctz((unsigned)a.blocks_per_wg);
    const int wgb0 = (int)(blockIdx.x >> a.ks_shift);
    for (int t = wave; t < (rounds << bshift); t += waves) {
      const int r = t >> bshift, b = t & (a.blocks_per_wg - 1);
      const int rb = (wgb0 + r * wg_stride) * a.blocks_per_wg + b;
      if (rb >= a.nblocks) continue;  // wave-uniform
      const float* tiles = partial + (size_t)(r * waves + b * a.kw) * (MT * 256);
      float4_t sum[MT];
#pragma unroll
      for (int t = 0; t < MT; ++t) sum[t] = (float4_t){0.f, 0.f, 0.f, 0.f};
      for (int w = 0; w < a.kw; ++w) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
          for (int q = 0; q < 4; ++q) sum[t][q] += tiles[(w * MT + t) * 256 + (4 * g + q) * 16 + nl];
      }
      emit(rb, sum);
    }
  }
}


template <int FMT, bool WIDE, bool GROUP, int MT>
int launch_mfma_u(int unroll, const MfmaArgs& a, int grid, int threads, size_t lds_bytes, hipStream_t stream) {
  // 16 waves leave 128 registers per lane: enough for one or two iterations in flight
  // (and for one tile of activation rows: more tiles come with at most 8 waves)
  const void* fn;
  if (threads > 512) {
    if constexpr (MT > 1) {
      return set_error(TLHIP_ERR_INVALID, "gemv_mfma: more than 16 activation rows take at most 8 waves per workgroup");
    } else {
      fn = unroll == 1 ? (const void*)gemv_mfma_kernel<FMT, 1, WIDE, 1024, false, GROUP>
                       : (const void*)gemv_mfma_kernel<FMT, 2, WIDE, 1024, false, GROUP>;
    }
  } else {
    switch (unroll) {
      case 1: fn = (const void*)gemv_mfma_kernel<FMT, 1, WIDE, 512, false, GROUP, MT>; break;
      case 2: fn = (const void*)gemv_mfma_kernel<FMT, 2, WIDE, 512, false, GROUP, MT>; break;
      default: fn = (const void*)gemv_mfma_kernel<FMT, 4, WIDE, 512, false, GROUP, MT>; break;
    }
  }
  void* args[] = {(void*)&a};
  return launch_kernel(fn, dim3(grid), dim3(threads), args, lds_bytes, stream);
}

// The form with whole-line weight loads (2 or 4 iterations in flight).
template <int FMT, bool WIDE, bool GROUP, int MT>
int launch_mfma_line(int unroll, const MfmaArgs& a, int grid, int threads, size_t lds_bytes, hipStream_t stream) {
  const void* fn;
  if (threads > 512) {
    if constexpr (MT > 1) {
      return set_error(TLHIP_ERR_INVALID, "gemv_mfma: more than 16 activation rows take at most 8 waves per workgroup");
    } else {
      fn = (const void*)gemv_mfma_kernel<FMT, 2, WIDE, 1024, true, GROUP>;
    }
  } else if (unroll == 2) {
    fn = (const void*)gemv_mfma_kernel<FMT, 2, WIDE, 512, true, GROUP, MT>;
  } else {
    fn = (const void*)gemv_mfma_kernel<FMT, 4, WIDE, 512, true, GROUP, MT>;
  }
  void* args[] = {(void*)&a};
  return launch_kernel(fn, dim3(grid), dim3(threads), args, lds_bytes, stream);
}

// Kernel instance for (format, group size, K, configuration): the scale loads are wide
// wherever a batch's scales are contiguous and aligned.
template <bool GROUP, int MT = 1>
int launch_mfma_instance(int format, int group_size, int64_t k, int unroll, int line, const MfmaArgs& a, int grid,
                         int threads, size_t lds_bytes, hipStream_t stream) {
  switch (format) {
    case TLHIP_FMT_INT4_GROUPED:
      // one scale per 16-byte chunk and 16-byte aligned scale vectors: wide scale loads
      if (line == 1)  // group size 32 and K % 256 == 0: the wide scale loads as well
        return launch_mfma_line<TLHIP_FMT_INT4_GROUPED, true, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
      if (group_size == 32 && (unroll == 1 || k % 256 == 0))
        return launch_mfma_u<TLHIP_FMT_INT4_GROUPED, true, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
      return launch_mfma_u<TLHIP_FMT_INT4_GROUPED, false, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
    case TLHIP_FMT_INT8_GROUPED:
      if (line == 1 && group_size == 64)  // one scale per iteration: the wide scale loads as well
        return launch_mfma_line<TLHIP_FMT_INT8_GROUPED, true, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
      if (line == 1) return launch_mfma_line<TLHIP_FMT_INT8_GROUPED, false, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
      return launch_mfma_u<TLHIP_FMT_INT8_GROUPED, false, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
    default:
      if (line == 1) return launch_mfma_line<TLHIP_FMT_INT8_ROW, false, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
      return launch_mfma_u<TLHIP_FMT_INT8_ROW, false, GROUP, MT>(unroll, a, grid, threads, lds_bytes, stream);
  }
}

// Every instance launch_mfma_instance can reach, in prepare mode (see launch_kernel).
template <bool GROUP, int MT = 1>
int prepare_mfma_instances() {
  MfmaArgs a;
  memset(&a, 0, sizeof a);
  for (int threads : {512, 1024})
    for (int unroll : {1, 2, 4}) {
      if (threads == 1024 && (unroll == 4 || MT > 1)) continue;
      int rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT4_GROUPED, 32, 256, unroll, 0, a, 1, threads, 0, nullptr);
      if (!rc) rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT4_GROUPED, 64, 256, unroll, 0, a, 1, threads, 0, nullptr);
      if (!rc) rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT8_GROUPED, 128, 256, unroll, 0, a, 1, threads, 0, nullptr);
      if (!rc) rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT8_ROW, 0, 256, unroll, 0, a, 1, threads, 0, nullptr);
      if (unroll != 1) {
        if (!rc) rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT4_GROUPED, 32, 256, unroll, 1, a, 1, threads, 0, nullptr);
        if (!rc) rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT8_GROUPED, 64, 256, unroll, 1, a, 1, threads, 0, nullptr);
        if (!rc) rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT8_GROUPED, 128, 256, unroll, 1, a, 1, threads, 0, nullptr);
        if (!rc) rc = launch_mfma_instance<GROUP, MT>(TLHIP_FMT_INT8_ROW, 0, 256, unroll, 1, a, 1, threads, 0, nullptr);
      }
      if (rc) return rc;
    }
  return TLHIP_OK;
}

}  // namespace

// One launch through the single-problem instances (gemv_mfma.hip) or the instances with a
// problem table (gemv_mfma_group.hip): two translation units, compiled side by side.
int launch_mfma_single(int format, int group_size, int64_t k, int unroll, int line, const MfmaArgs& a, int grid, int threads,
                       size_t lds_bytes, hipStream_t stream);
int launch_mfma_grouped(int format, int group_size, int64_t k, int unroll, int line, const MfmaArgs& a, int grid, int threads,
                        size_t lds_bytes, hipStream_t stream);
int prepare_mfma_single();
int prepare_mfma_grouped();
// The instances for 17..64 activation rows (`tiles` = 2 or 4 tiles of 16 rows), single
// problem, at most 8 waves per workgroup: gemv_mfma_rows.hip.
int launch_mfma_rows(int tiles, int format, int group_size, int64_t k, int unroll, int line, const MfmaArgs& a, int grid,
                     int threads, size_t lds_bytes, hipStream_t stream);
int prepare_mfma_rows();

}  // namespace tlhip
