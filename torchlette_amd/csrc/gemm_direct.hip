// Prefill GEMM over packed weights, second form: the weights stay PACKED until they
// are in the operand registers.  Y[M,N] = epilogue(alpha * X[M,K] * W[N,K]^T); same
// contract and reference route as gemm_prefill.hip
// (src/backend/webgpu/ops/matmul-ops.ts:163-181;
// src/schedule/matmul-skeleton.ts:738-966).  Written for int4 in groups, described
// below; the int8 forms (groups of 64 or more, and one scale per row) are the same
// pipeline on 128 bytes per row and step, described at the kernel's template flags.
//
// Why a second form: with the dequantised f16 weights staged through LDS a tile
// moves about 1 KB of LDS traffic per MFMA and the kernel is bound by LDS, not
// by the matrix cores.  Here, per 128-k step of a BM x BN tile,
//   * the packed weights (BN rows x 64 bytes) go global -> registers -> LDS as
//     they are, 16 bytes per lane with four consecutive lanes on one row, so the
//     global loads are coalesced (a lane loading its own MFMA operand row made
//     64 scattered 16-byte requests per instruction and cost a quarter of the
//     kernel's time); LDS holds them with the chunk position XOR-swizzled by
//     the row so that the operand reads spread over all banks;
//   * a lane of the B operand of v_mfma_f32_32x32x16_f16 (weight row n, k half
//     lk) reads ITS two 16-byte chunks (64 weights) from LDS and dequantises them
//     in registers, one 32-bit word (8 weights, one MFMA) at a time: exact
//     integers in f16, times the group scale (loaded by the lane itself, 4
//     bytes per step), one rounding.  LDS traffic for W is a quarter of what
//     dequantised f16 would be;
//   * the k order inside a step is chosen to fit that: MFMA (c, w) of a step
//     covers k = 64*lk + 32*c + 8*w + (0..7) for lane half lk, and the A operand
//     reads the activations of exactly those k from LDS;
//   * X goes global -> registers -> LDS in parts spread over the step, written
//     with the (0,4,1,5,2,6,3,7) order the int4 unpack produces.  LDS holds HALF a
//     step of X twice: the MFMA groups 0..3 of a step read the k-columns
//     {0..3, 8..11} (16-byte units of the 128-k row), the groups 4..7 the columns
//     {4..7, 12..15}; while one half is read the other is written (the second half
//     of this step during its first half, the first half of the next step during
//     its second half), and the two LDS-only barriers of a step - in the middle
//     and at the end - are what the single W buffer needs anyway.  A 128-row tile
//     with a 256-row W buffer takes 48 KB, so two workgroups share a CU;
//   * 4 or 8 waves per workgroup, two waves per SIMD resident.
// MFMA-bound by design: per MFMA a wave reads 1 KB / TN from LDS and spends
// 14 / TM VALU instructions on dequantisation.
#include <cstring>
#include <type_traits>
#include <utility>

#include "gemm_common.h"

namespace tlhip {
namespace {

constexpr int DK = 128;            // k per step
// LDS row of half a step of X: 8 units of 16 bytes, the unit column XOR-ed with bits
// 1..3 of the row, so that the 16 lanes of an A operand read (16 rows, one column)
// fall on 16 different bank groups.
constexpr int HROW_UNITS = 8;

struct DirectArgs {
  const uint8_t* packed;  // row stride K/2 bytes
  const uint16_t* scales; // f16 bits, K/G per row
  const _Float16* x;
  int m, n, k;
  int w_row_bytes;
  int cpg_shift;          // log2(16-byte chunks per scale group)
  int groups_per_row;
  int ksteps;             // K / 128
  int ksplit;             // workgroups that share a tile, each walking ksteps / ksplit steps of K (1 = none)
  float* workspace;       // ksplit > 1: the slices' partial sums, [slice][M][N] f32
  TileMap map;
  OutArgs out;
};

// The epilogue of a wave's TM row blocks of 32 rows, one call each.
template <int TN, bool ROW, int... I>
__device__ __forceinline__ void epilogue_of_row_blocks(std::integer_sequence<int, I...>, float* patch,
                                                       const float16_t (&acc)[sizeof...(I)][TN], int lane, int row0, int col0,
                                                       const OutArgs& o, float* plane) {
  (wave_epilogue<TN, true, ROW>(patch, acc[I], lane, row0 + I * 32, col0, o, plane), ...);
}

// WM x WN waves, each owning TM x TN MFMA tiles of 32 x 32.  G32: one scale per
// 16-byte chunk (group size 32), the two scales of a lane's step come as one
// 4-byte load.
// I8: int8 weights with one f16 scale per group of 64 or more (the reference's own
// format).  A 128-k step of a row is 128 bytes = 8 chunks; a lane of the B operand reads
// the 4 chunks of its k half and turns two words (8 weights) into an MFMA operand, in
// natural k order (k = 64*lk + 8*kk for MFMA group kk: the same activation units as for
// int4, without the int4 order inside a unit); the 1/127 of the format rides on alpha.
// ROW (with I8): int8 weights with one f32 scale per row.  The operand is the bare integer
// (exact in f16, no multiplication, no scale loads in the loop) and the row's scale
// multiplies the sums in the epilogue, as a factor per output column.
template <int WM, int WN, int TM, int TN, bool G32, bool I8 = false, bool ROW = false>
__global__ __launch_bounds__(WM * WN * 64, (TM * TN >= 16 ? 1 : 2)) void gemm_direct_kernel(const DirectArgs a) {
  static_assert(!(G32 && I8), "int8 groups are 64 weights or more");
  static_assert(!ROW || I8, "per-row scales are an int8 format");
  constexpr int THREADS = WM * WN * 64;
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int CPR = I8 ? 8 : 4;             // 16-byte chunks of a weight row per step
  constexpr int X_LOADS = BM * 16 / THREADS;  // 16-byte units of the X tile per thread per step
  constexpr int W_LOADS = BN * CPR / THREADS; // 16-byte chunks of the W tile per thread per step
  static_assert(BM * 16 % THREADS == 0 && BN * CPR % THREADS == 0, "tiles must divide over the threads");
  constexpr int X_UNITS = BM * HROW_UNITS;  // half a step of the X tile
  // The 256x128 tile of eight 128x32 waves issues its MFMA groups at raised priority,
  // so that the wave it shares a SIMD with (same workgroup, same barriers, the same
  // phase of the step) does not delay them with its dequantisation: measured 2.5-3.5 %
  // faster at M = 512..8192.  Every other tile measured 2-7 % SLOWER with the same two
  // instructions (the four-wave tiles whichever way round the priorities are), so they
  // stay without.
  constexpr bool MFMA_PRIO = WM == 2 && WN == 4 && TM == 4 && TN == 1;
  extern __shared__ u32x4 lds[];  // X first half, X second half, W buffer
  u32x4* const lds_w = lds + 2 * X_UNITS;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int lrow = lane & 31, lk = lane >> 5;

  // K split across workgroups: the ksplit workgroups of consecutive ids take the slices of
  // one tile and leave their partial sums in the workspace (a second launch adds them).  A
  // launch of a few tiles (M of a few hundred rows on a decode-sized matrix) would leave
  // most CUs idle while each workgroup walks all of K on its own.
  const int slice = a.ksplit > 1 ? (int)(blockIdx.x % (unsigned)a.ksplit) : 0;
  const int tile_id = a.ksplit > 1 ? (int)(blockIdx.x / (unsigned)a.ksplit) : (int)blockIdx.x;
  const int nsteps = a.ksteps / a.ksplit;  // steps of this workgroup
  const int step0 = slice * nsteps;        // its first step of K
  int tm_idx, tn_idx;
  if (!tile_of(a.map, tile_id, tm_idx, tn_idx)) return;  // padding of the tile map (whole workgroup)
  const int m0 = tm_idx * BM, n0 = tn_idx * BN;

  // ---- W: global -> registers -> LDS, packed --------------------------------
  // chunk q = tid + i*THREADS of the tile: row q/4, chunk q%4 of the step's 64 bytes
  u32x4 wr[W_LOADS];
  auto load_w = [&](int step) {
    const int st = step0 + min(step, nsteps - 1);  // past the end: a harmless reload of the last step
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      const int q = tid + i * THREADS;
      const int row = min(n0 + q / CPR, a.n - 1);
      wr[i] = *(const u32x4*)(a.packed + (size_t)row * a.w_row_bytes + (size_t)st * (CPR * 16) + (q % CPR) * 16);
    }
  };
  auto store_w = [&]() {
    u32x4* ws = lds_w;
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      const int q = tid + i * THREADS;
      const int r = q / CPR;
      if constexpr (I8) ws[r * 8 + ((q & 7) ^ (r & 7))] = wr[i];
      else ws[r * 4 + ((q & 3) ^ ((r >> 2) & 3))] = wr[i];
    }
  };
  // The lane's scales: raw bits, two stages (this step, next step).
  const uint16_t* sptr[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int row = min(n0 + (wn * TN + j) * 32 + lrow, a.n - 1);
    sptr[j] = a.scales + (size_t)row * a.groups_per_row;
  }
  struct Scales {
    uint32_t s[TN][2];  // G32: s[j][0] holds both scales; else one 16-bit scale each
  };
  auto load_s = [&](int step, Scales& sc) {
    if constexpr (ROW) return;
    const int st = step0 + min(step, nsteps - 1);
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      if (G32) {
        sc.s[j][0] = *(const uint32_t*)(sptr[j] + st * 4 + lk * 2);
      } else {
        const int ch = st * 4 + lk * 2;
        sc.s[j][0] = sptr[j][ch >> a.cpg_shift];
        sc.s[j][1] = sptr[j][(ch + 1) >> a.cpg_shift];
      }
    }
  };

  // ---- X: global -> registers -> LDS, two parts per half step -----------------------
  // unit u of a half: row u / 8, column c = u % 8 = 4 * lk + j, which is unit
  // 8 * lk + 4 * half + j of the step's 128-k row
  static_assert(X_LOADS % 4 == 0, "X tile units per thread must divide into four staging parts");
  constexpr int XH = X_LOADS / 4;
  u32x4 xr[XH];
  auto load_x = [&](int step, int half, int part) {
    const int k0 = (step0 + min(step, nsteps - 1)) * DK;
#pragma unroll
    for (int i = 0; i < XH; ++i) {
      const int u = tid + (part * XH + i) * THREADS;
      const int row = min(m0 + (u >> 3), a.m - 1);
      const int c = u & 7;
      xr[i] = *(const u32x4*)(a.x + (size_t)row * a.k + k0 + ((c >> 2) * 8 + half * 4 + (c & 3)) * 8);
    }
  };
  auto store_x = [&](int half, int part) {
    u32x4* xs = lds + half * X_UNITS;
#pragma unroll
    for (int i = 0; i < XH; ++i) {
      const int u = tid + (part * XH + i) * THREADS;
      const int r = u >> 3, c = u & 7;
      xs[r * HROW_UNITS + (c ^ ((r >> 1) & 7))] = I8 ? xr[i] : permute_x_for_int4(xr[i]);
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // ---- operands ------------------------------------------------------------------
  // One step = 8 MFMA groups kk = 4*c + w, software pipelined by hand.  While the
  // MFMAs of group kk run, the B operands of group kk+1 are dequantised into the
  // other of two operand sets, and each A operand is re-read from LDS for group
  // kk+1 as soon as its last MFMA of group kk has been issued: an MFMA occupies
  // the matrix pipe for 8 passes and the wave can issue 7 other instructions
  // meanwhile, so the dequantisation and the LDS reads hide under the MFMAs.
  // the lane's packed chunks of the step.  int4: c = 0, 1.  int8: four chunks through two
  // register slots: chunks 0 and 1 at the top of the step, chunk 2 into slot 0 once MFMA
  // group 1 has been dequantised (the last user of chunk 0), chunk 3 into slot 1 behind
  // group 3; all four are read before the mid-step barrier that frees the W buffer.
  u32x4 bw[TN][2];
  auto read_w = [&](int c) {
    const u32x4* ws = lds_w;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int r = (wn * TN + j) * 32 + lrow;
      if constexpr (I8) bw[j][c & 1] = ws[r * 8 + ((lk * 4 + c) ^ (r & 7))];
      else bw[j][c] = ws[r * 4 + ((lk * 2 + c) ^ ((r >> 2) & 3))];
    }
  };
  auto dequant = [&](const Scales& sc, int kk, half8_t (&bf)[TN]) {
    const int c = kk >> 2, w = kk & 3;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t bits = ROW ? 0x3c00u : (G32 ? (c ? (sc.s[j][0] >> 16) : (sc.s[j][0] & 0xffffu)) : sc.s[j][c]);
      const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)bits);
      const half2_t s2 = {sh, sh};
      half2_t h[4];
      if constexpr (I8) {
        // chunk kk / 2 of the lane's four, its words 0, 1 (kk even) or 2, 3 (kk odd)
        const u32x4 chunk8 = bw[j][(kk >> 1) & 1];
        unpack_int8_word((kk & 1) ? chunk8.z : chunk8.x, h);
        unpack_int8_word((kk & 1) ? chunk8.w : chunk8.y, h + 2);
      } else {
        const u32x4 chunk = bw[j][c];
        const uint32_t word = w == 0 ? chunk.x : (w == 1 ? chunk.y : (w == 2 ? chunk.z : chunk.w));
        unpack_int4_word(word, h);
      }
      half8_t v;
      const half2_t h0 = ROW ? h[0] : h[0] * s2, h1 = ROW ? h[1] : h[1] * s2, h2 = ROW ? h[2] : h[2] * s2,
                    h3 = ROW ? h[3] : h[3] * s2;
      v[0] = h0[0]; v[1] = h0[1]; v[2] = h1[0]; v[3] = h1[1];
      v[4] = h2[0]; v[5] = h2[1]; v[6] = h3[0]; v[7] = h3[1];
      bf[j] = v;
    }
  };
  half8_t af[TM];
  // group kk reads column 4 * lk + kk % 4 of half kk / 4; the row's swizzle term is
  // (lrow >> 1) & 7 (the other terms of the row are multiples of 32)
  const int acol = (lk * 4) ^ ((lrow >> 1) & 7);
  auto read_a = [&](int kk, int i) {
    const u32x4* xs = lds + (kk >> 2) * X_UNITS + (wm * TM * 32 + lrow) * HROW_UNITS + (acol ^ (kk & 3));
    af[i] = __builtin_bit_cast(half8_t, xs[i * 32 * HROW_UNITS]);
  };
  // MFMAs of one group; `next` >= 0: re-read each A operand for group `next`
  auto group = [&](const half8_t (&bf)[TN], int next) {
    if constexpr (MFMA_PRIO) __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
      if (next >= 0) read_a(next, i);
    }
    if constexpr (MFMA_PRIO) __builtin_amdgcn_s_setprio(0);
  };

  // ---- pipeline -----------------------------------------------------------------
  // W of step s+1 and the halves of X are loaded to registers while step s computes
  // and go to LDS before the barrier behind which they are read; the scales are one
  // more step ahead.  Every load is unconditional (clamped past the end).
  Scales s0, s1;
  half8_t bfA[TN], bfB[TN];
  load_s(0, s0);
  load_s(1, s1);
  load_w(0);
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    load_x(0, 0, p);
    store_x(0, p);
  }
  store_w();
  lds_barrier();
  // The scheduling fences keep the compiler from sinking the global loads to
  // their use (the LDS store), which would expose their latency.
  // CARRY (wave tiles two or more MFMA tiles wide): the two barriers of a step sit one
  // MFMA group EARLIER than the data needs them.  Group 3 is issued behind the mid-step
  // barrier and group 7 behind the end barrier, at the top of the next step, so that
  // the LDS reads (and, at the top of a step, the first dequantisation) that can only
  // start behind a barrier run under a group of MFMAs instead of an idle matrix pipe:
  // 1-3 % faster in an A/B within one run.  The one-tile-wide waves (four MFMAs to a
  // group) measured 2-3 % slower that way and keep every group in front of its barrier.
  constexpr bool CARRY = TN >= 2;
  auto step = [&](int s, Scales& sc, auto has_prev) {
    load_w(s + 1);
    load_x(s, 1, 0);
    read_w(0);
    read_w(1);
    if constexpr (CARRY && decltype(has_prev)::value) {
      dequant(sc, 0, bfA); group(bfB, 0);  // group 7 of the step before
    } else {
#pragma unroll
      for (int i = 0; i < TM; ++i) read_a(0, i);
      dequant(sc, 0, bfA);
    }
    __builtin_amdgcn_sched_barrier(0);
    dequant(sc, 1, bfB);
    if constexpr (I8) read_w(2);
    group(bfA, 1);
    dequant(sc, 2, bfA); group(bfB, 2);
    __builtin_amdgcn_sched_barrier(0);
    store_x(1, 0);
    load_x(s, 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    dequant(sc, 3, bfB);
    if constexpr (I8) read_w(3);
    group(bfA, 3);
    if constexpr (!CARRY) {
      // group 3 re-reads nothing: the second half of X is whole only behind the barrier
      dequant(sc, 4, bfA); group(bfB, -1);
    }
    __builtin_amdgcn_sched_barrier(0);
    store_x(1, 1);
    load_x(s + 1, 0, 0);
    // the barrier also frees the single W buffer: every wave took its chunks of this
    // step at the top of the step
    lds_barrier();
    store_w();
    if constexpr (CARRY) {
      dequant(sc, 4, bfA); group(bfB, 4);
    } else {
#pragma unroll
      for (int i = 0; i < TM; ++i) read_a(4, i);
    }
    __builtin_amdgcn_sched_barrier(0);
    dequant(sc, 5, bfB); group(bfA, 5);
    dequant(sc, 6, bfA); group(bfB, 6);
    __builtin_amdgcn_sched_barrier(0);
    store_x(0, 0);
    load_x(s + 1, 0, 1);
    __builtin_amdgcn_sched_barrier(0);
    dequant(sc, 7, bfB); group(bfA, 7);
    if constexpr (!CARRY) group(bfB, -1);
    __builtin_amdgcn_sched_barrier(0);
    load_s(s + 2, sc);
    store_x(0, 1);
    lds_barrier();
  };
  // The first step on its own (nothing to carry in), then whole pairs in the loop and
  // the odd step after it: a step under a branch inside the loop would make the wait
  // counters at the loop head pessimistic.
  step(0, s0, std::false_type{});
  int s = 1;
  for (; s + 1 < nsteps; s += 2) {
    step(s, s1, std::true_type{});
    step(s + 1, s0, std::true_type{});
  }
  if (s < nsteps) step(s, s1, std::true_type{});
  if constexpr (CARRY) group(bfB, -1);  // group 7 of the last step

  // Epilogue: one 32-row block of the wave at a time through a private LDS patch
  // (the staging buffers are free after the last barrier).
  float* patch = (float*)lds + wave * (32 * (TN * 32 + 4));
  // a K slice leaves its bare partial sums, f32, row-major, in this slice's M x N plane of
  // the workspace; the reduce launch adds the planes in slice order and runs the epilogue
  float* const plane = a.ksplit > 1 ? a.workspace + (size_t)slice * a.m * a.n : nullptr;
  // One call per row block, written out at compile time (a loop here is only unrolled while
  // its unrolled size stays under the compiler's threshold; left as a loop it indexes the
  // accumulators at run time, and they move to scratch memory for the whole kernel).
  epilogue_of_row_blocks<TN, ROW>(std::make_integer_sequence<int, TM>{}, patch, acc, lane, m0 + wm * TM * 32, n0 + wn * TN * 32,
                                  a.out, plane);
}

// v[e] = ops(alpha * v[e]) for the W consecutive columns from `col` on (output elements
// from `idx` on); W = 8: whole 16-byte pieces of the inputs, W = 1: one element.
template <int W>
__device__ __forceinline__ void apply_epilogue_scaled(const OutArgs& o, float (&v)[W], int64_t col, int64_t idx) {
#pragma unroll
  for (int e = 0; e < W; ++e) v[e] *= o.col_scale ? o.alpha * o.col_scale[col + e] : o.alpha;
  if constexpr (W == 8) {
    apply_epilogue_row8(o.epi, v, col, idx, true, o.n - 1);
  } else {
#pragma unroll
    for (int e = 0; e < W; ++e) v[e] = apply_epilogue(o.epi, v[e], col + e, idx + e);
  }
}

// Second launch of a K-sliced GEMM: y = epilogue(alpha * sum over the slices' planes, in
// slice order).  A reduction by the last workgroup to arrive for a tile (one launch) was
// built first and cost 12 us + 1.6 us per slice: one CU reading up to 512 KB of partial
// tiles with device-scope loads.  Here every CU takes its share, the kernel boundary orders
// the planes' stores before these loads, and the sum is the same from launch to launch.
// VEC: 8 consecutive columns per thread (N % 8 == 0, y 16-byte aligned), else one element.
template <bool VEC, int KS>
__global__ __launch_bounds__(256) void direct_reduce_kernel(const float* __restrict__ planes, const OutArgs o) {
  const int64_t plane = (int64_t)o.m * o.n;
  const int64_t idx = ((int64_t)blockIdx.x * 256 + threadIdx.x) * (VEC ? 8 : 1);
  if (idx >= plane) return;
  constexpr int W = VEC ? 8 : 1;
  // every plane's loads issued before the first is added (a loop over a run-time slice
  // count made each plane a round trip to memory of its own)
  float part[KS][W];
#pragma unroll
  for (int sl = 0; sl < KS; ++sl) {
    const float* src = planes + sl * plane + idx;
    if constexpr (VEC) {
      const float4_t a0 = __builtin_nontemporal_load((const float4_t*)src);
      const float4_t a1 = __builtin_nontemporal_load((const float4_t*)(src + 4));
      part[sl][0] = a0[0]; part[sl][1] = a0[1]; part[sl][2] = a0[2]; part[sl][3] = a0[3];
      part[sl][W - 4] = a1[0]; part[sl][W - 3] = a1[1]; part[sl][W - 2] = a1[2]; part[sl][W - 1] = a1[3];
    } else {
      part[sl][0] = __builtin_nontemporal_load(src);
    }
  }
  float v[W];
#pragma unroll
  for (int e = 0; e < W; ++e) {
    v[e] = 0.f;
#pragma unroll
    for (int sl = 0; sl < KS; ++sl) v[e] += part[sl][e];  // slice order
  }
  const int64_t col = idx % o.n;
  apply_epilogue_scaled(o, v, col, idx);
  if constexpr (VEC) {
    if (o.y_dtype == TLHIP_F16) {
      half8_t h;
#pragma unroll
      for (int e = 0; e < W; ++e) h[e] = (_Float16)v[e];
      *(half8_t*)((_Float16*)o.y + idx) = h;
    } else {
      float* dst = (float*)o.y + idx;
      *(float4_t*)dst = (float4_t){v[0], v[1], v[2], v[3]};
      *(float4_t*)(dst + 4) = (float4_t){v[W - 4], v[W - 3], v[W - 2], v[W - 1]};
    }
  } else {
    store_out(o.y, o.y_dtype, idx, v[0]);
  }
}

template <bool VEC>
int launch_direct_reduce(int ks, unsigned grid, const float* planes, const OutArgs& o, hipStream_t stream) {
  switch (ks) {
    case 2: hipLaunchKernelGGL((direct_reduce_kernel<VEC, 2>), dim3(grid), dim3(256), 0, stream, planes, o); break;
    case 4: hipLaunchKernelGGL((direct_reduce_kernel<VEC, 4>), dim3(grid), dim3(256), 0, stream, planes, o); break;
    case 8: hipLaunchKernelGGL((direct_reduce_kernel<VEC, 8>), dim3(grid), dim3(256), 0, stream, planes, o); break;
    default: hipLaunchKernelGGL((direct_reduce_kernel<VEC, 16>), dim3(grid), dim3(256), 0, stream, planes, o); break;
  }
  return TLHIP_OK;
}

// The tiles built for int8 weights (the others would only lengthen the build).
template <int WM, int WN, int TM, int TN>
constexpr bool kInt8Tile = (WM == 2 && WN == 2 && TM == 2 && TN == 2) || (WM == 2 && WN == 4 && TM == 2 && TN == 2) ||
                           (WM == 2 && WN == 4 && TM == 4 && TN == 1) || (WM == 2 && WN == 4 && TM == 4 && TN == 2);

template <int WM, int WN, int TM, int TN>
int launch_direct_tile(const DirectArgs& a, bool g32, bool int8, hipStream_t stream) {
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  const void* fn = g32 ? (const void*)gemm_direct_kernel<WM, WN, TM, TN, true>
                       : (const void*)gemm_direct_kernel<WM, WN, TM, TN, false>;
  if (int8) {
    if constexpr (kInt8Tile<WM, WN, TM, TN>)
      fn = a.out.col_scale ? (const void*)gemm_direct_kernel<WM, WN, TM, TN, false, true, true>
                           : (const void*)gemm_direct_kernel<WM, WN, TM, TN, false, true>;
    else return set_error(TLHIP_ERR_INVALID, "gemm_direct: this tile is not built for int8 weights");
  }
  size_t lds_bytes = (size_t)(2 * BM * HROW_UNITS + BN * (int8 ? 8 : 4)) * 16;
  const size_t patch_bytes = (size_t)WM * WN * 32 * (TN * 32 + 4) * sizeof(float);
  if (lds_bytes < patch_bytes) lds_bytes = patch_bytes;
  DirectArgs b = a;
  int grid = 0;
  b.map = make_tile_map((a.m + BM - 1) / BM, (a.n + BN - 1) / BN, TileCost{BM * 2, int8 ? BN : BN / 2}, &grid);
  void* args[] = {(void*)&b};
  return launch_kernel(fn, dim3(grid * (a.ksplit > 1 ? a.ksplit : 1)), dim3(WM * WN * 64), args, lds_bytes, stream);
}

struct DirectTile {
  int bm, bn, wm, wn;
};
// tile M, tile N, waves M, waves N
constexpr DirectTile kDirectTiles[] = {
    {256, 256, 2, 4},  // wave tile 128 x 64
    {256, 128, 2, 4},  // wave tile 128 x 32
    {128, 256, 2, 4},  // wave tile 64 x 64
    {256, 128, 4, 2},  // wave tile 64 x 64
    {128, 128, 2, 2},  // wave tile 64 x 64, 4 waves: two workgroups share a CU
    {256, 256, 2, 2},  // wave tile 128 x 128, 4 waves, one per SIMD
    {128, 256, 1, 4},  // wave tile 128 x 64, 4 waves, 48 KB of LDS: two workgroups share a CU
    {128, 192, 2, 2},  // wave tile 64 x 96, 4 waves: M = 512 x N = 12288 makes exactly 256 tiles, one per CU
};

}  // namespace

// y = epilogue(alpha * sum of the `ks` planes of o.m x o.n f32 partial sums at `planes`),
// enqueued behind the launch that wrote them: the second launch of a K-sliced tiled GEMM.
int launch_k_slice_reduce(int ks, const float* planes, const OutArgs& o, hipStream_t stream) {
  const bool vec = o.vec_ok;
  const int64_t threads = ((int64_t)o.m * o.n + (vec ? 7 : 0)) / (vec ? 8 : 1);
  const unsigned grid = (unsigned)((threads + 255) / 256);
  if (vec) launch_direct_reduce<true>(ks, grid, planes, o, stream);
  else launch_direct_reduce<false>(ks, grid, planes, o, stream);
  TLHIP_CHECK_HIP(hipGetLastError());
  return TLHIP_OK;
}

bool gemm_direct_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  static const char* reasons[] = {
      "not the tiled_direct variant",
      "weights must be int4-grouped, or int8-row or int8-grouped with a group size that is a multiple of 64 on one of the tiles "
      "128x128 2x2, 128x256 2x4, 256x128 2x4, 256x256 2x4",
      "activations must be f16",
      "K must be a multiple of 128",
      "group size must be a multiple of 32",
      "K split across workgroups (p5) must be 0, 1 or a power of two up to 16 that divides K / 128, with the slices' "
      "partial sums (p5 x M x N, f32) inside the library's workspace",
      "tile (M, N, waves M, waves N) must be one of 256x256 2x4, 256x128 2x4, 128x256 2x4, 256x128 4x2, 128x128 2x2, 256x256 2x2, 128x256 1x4, 128x192 2x2 with tile K 128",
  };
  auto fail = [&](int i) {
    if (why) *why = reasons[i];
    return false;
  };
  if (c.variant != VARIANT_TILED_DIRECT) return fail(0);
  const bool row = p.format == TLHIP_FMT_INT8_ROW;
  const bool int8 = p.format == TLHIP_FMT_INT8_GROUPED || row;
  if (p.format != TLHIP_FMT_INT4_GROUPED && !int8) return fail(1);
  if (int8) {
    const bool tile_ok = (c.p0 == 128 && c.p1 == 128 && c.p3 == 2 && c.p4 == 2) || (c.p0 == 128 && c.p1 == 256 && c.p3 == 2 && c.p4 == 4) ||
                         (c.p0 == 256 && c.p1 == 128 && c.p3 == 2 && c.p4 == 4) || (c.p0 == 256 && c.p1 == 256 && c.p3 == 2 && c.p4 == 4);
    if ((!row && p.group_size % 64 != 0) || !tile_ok) return fail(1);
  }
  if (p.x_dtype != TLHIP_F16) return fail(2);
  if (p.k % DK != 0 || p.k == 0) return fail(3);
  if (!row && p.group_size % 32 != 0) return fail(4);
  if (c.p2 != DK) return fail(6);
  for (const auto& t : kDirectTiles)
    if (t.bm == c.p0 && t.bn == c.p1 && t.wm == c.p3 && t.wn == c.p4) {
      const int ks = c.p5 < 1 ? 1 : c.p5;
      if (ks > 1) {
        if (ks > 16 || (ks & (ks - 1)) != 0 || (p.k / DK) % ks != 0) return fail(5);
        if ((size_t)p.m * (size_t)p.n * ks > kSplitWorkspaceFloats) return fail(5);
      }
      return true;
    }
  return fail(6);
}

int launch_gemm_direct(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemm_direct_config_applicable(p, c, &why))
    return set_error(TLHIP_ERR_INVALID, "gemm_direct: config not applicable: %s", why);
  if (p.m == 0 || p.n == 0) return TLHIP_OK;
  DirectArgs a;
  a.packed = (const uint8_t*)p.packed;
  a.scales = (const uint16_t*)p.scales;
  a.x = (const _Float16*)p.x;
  a.m = (int)p.m;
  a.n = (int)p.n;
  a.k = (int)p.k;
  const bool row = p.format == TLHIP_FMT_INT8_ROW;
  a.w_row_bytes = (int)(p.format == TLHIP_FMT_INT4_GROUPED ? p.k / 2 : p.k);
  a.cpg_shift = row ? 0 : __builtin_ctz((unsigned)(p.group_size / 32));
  a.groups_per_row = row ? 0 : (int)(p.k / p.group_size);
  a.ksteps = (int)(p.k / DK);
  a.ksplit = c.p5 < 1 ? 1 : c.p5;
  a.workspace = nullptr;
  if (a.ksplit > 1) {
    int* counters = nullptr;  // this kernel combines its slices in a second launch, not by arrival
    const int rc = split_workspace(stream, &a.workspace, &counters);
    if (rc) return rc;
  }
  a.out.y = p.y;
  a.out.y_dtype = p.y_dtype;
  a.out.vec_ok = (p.n % 8 == 0) && ((uintptr_t)p.y % 16 == 0);
  a.out.m = (int)p.m;
  a.out.n = (int)p.n;
  a.out.alpha = p.alpha;
  a.out.epi = p.epi;
  a.out.col_scale = row ? (const float*)p.scales : nullptr;  // int8-row: w = q * scale[n], applied to the sums
  const bool int8 = p.format == TLHIP_FMT_INT8_GROUPED || row;
  const bool g32 = !int8 && p.group_size == 32;
  // the grouped format's 1/127 (quantize.ts: q = round(w / absmax * 127))
  if (p.format == TLHIP_FMT_INT8_GROUPED) a.out.alpha = p.alpha * (1.0f / 127.0f);
  int rc;
  if (c.p0 == 256 && c.p1 == 256 && c.p4 == 2) rc = launch_direct_tile<2, 2, 4, 4>(a, g32, int8, stream);
  else if (c.p0 == 256 && c.p1 == 256) rc = launch_direct_tile<2, 4, 4, 2>(a, g32, int8, stream);
  else if (c.p0 == 256 && c.p1 == 128 && c.p3 == 2) rc = launch_direct_tile<2, 4, 4, 1>(a, g32, int8, stream);
  else if (c.p0 == 128 && c.p1 == 256 && c.p3 == 1) rc = launch_direct_tile<1, 4, 4, 2>(a, g32, int8, stream);
  else if (c.p0 == 128 && c.p1 == 256) rc = launch_direct_tile<2, 4, 2, 2>(a, g32, int8, stream);
  else if (c.p0 == 128 && c.p1 == 128) rc = launch_direct_tile<2, 2, 2, 2>(a, g32, int8, stream);
  else if (c.p0 == 128 && c.p1 == 192) rc = launch_direct_tile<2, 2, 2, 3>(a, g32, int8, stream);
  else rc = launch_direct_tile<4, 2, 2, 2>(a, g32, int8, stream);
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  if (a.ksplit > 1) {
    const int rr = launch_k_slice_reduce(a.ksplit, a.workspace, a.out, stream);
    if (rr) return rr;
  }
  count_gemm_dispatch();
  return TLHIP_OK;
}

// Every instance launch_gemm_direct can reach, in prepare mode (see launch_kernel).
int prepare_gemm_direct_kernels() {
  DirectArgs a;
  memset(&a, 0, sizeof a);
  a.m = a.n = 1;
  a.ksplit = 1;
  for (bool g32 : {true, false}) {
    int rc = launch_direct_tile<2, 2, 4, 4>(a, g32, false, nullptr);
    if (!rc) rc = launch_direct_tile<2, 4, 4, 2>(a, g32, false, nullptr);
    if (!rc) rc = launch_direct_tile<2, 4, 4, 1>(a, g32, false, nullptr);
    if (!rc) rc = launch_direct_tile<1, 4, 4, 2>(a, g32, false, nullptr);
    if (!rc) rc = launch_direct_tile<2, 4, 2, 2>(a, g32, false, nullptr);
    if (!rc) rc = launch_direct_tile<2, 2, 2, 2>(a, g32, false, nullptr);
    if (!rc) rc = launch_direct_tile<2, 2, 2, 3>(a, g32, false, nullptr);
    if (!rc) rc = launch_direct_tile<4, 2, 2, 2>(a, g32, false, nullptr);
    if (rc) return rc;
  }
  static const float one = 1.f;
  for (const float* cs : {(const float*)nullptr, &one}) {  // int8 in groups, int8 per row
    a.out.col_scale = cs;
    int rc = launch_direct_tile<2, 2, 2, 2>(a, false, true, nullptr);
    if (!rc) rc = launch_direct_tile<2, 4, 2, 2>(a, false, true, nullptr);
    if (!rc) rc = launch_direct_tile<2, 4, 4, 1>(a, false, true, nullptr);
    if (!rc) rc = launch_direct_tile<2, 4, 4, 2>(a, false, true, nullptr);
    if (rc) return rc;
  }
  return TLHIP_OK;
}

}  // namespace tlhip
