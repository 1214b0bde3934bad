// Prefill GEMM over packed int4 weights, second form: the weight operand never
// touches LDS.  Y[M,N] = epilogue(alpha * X[M,K] * W[N,K]^T); same contract and
// reference route as gemm_prefill.hip (src/backend/webgpu/ops/matmul-ops.ts:163-181;
// src/schedule/matmul-skeleton.ts:738-966).
//
// Why a second form: with both operands staged through LDS a 4-wave tile moves
// about 1 KB of LDS traffic per MFMA and the kernel is bound by LDS, not by the
// matrix cores.  Here
//   * a lane of the B operand of v_mfma_f32_32x32x16_f16 (weight row n, k half
//     lk) loads ITS packed weights straight from global memory — 32 contiguous
//     bytes (two 16-byte chunks = 64 weights) per 128-k step, plus the two group
//     scales — and dequantises them in registers, one 32-bit word (8 weights,
//     one MFMA) at a time: exact integers in f16, times the scale, one rounding;
//   * the k order inside a step is chosen to fit that: MFMA (c, w) of a step
//     covers k = 64*lk + 32*c + 8*w + (0..7) for lane half lk, and the A operand
//     reads the activations of exactly those k from LDS;
//   * only X goes through LDS (global -> registers -> LDS in two halves per step,
//     double buffered, one LDS-only barrier per 128-k step), written with the
//     (0,4,1,5,2,6,3,7) order the int4 unpack produces;
//   * 8 waves (2 per SIMD) per workgroup, so one wave's dequantisation and LDS
//     reads overlap the other's MFMAs.
// MFMA-bound by design: per MFMA a wave reads 1 KB / TN from LDS and spends
// 14 / TM VALU instructions on dequantisation.
#include "gemm_common.h"

namespace tlhip {
namespace {

constexpr int DK = 128;            // k per step
constexpr int DROW_UNITS = 17;     // LDS row: 128 f16 = 16 units + 1 unit of padding

struct DirectArgs {
  const uint8_t* packed;  // row stride K/2 bytes
  const uint16_t* scales; // f16 bits, K/G per row
  const _Float16* x;
  int m, n, k;
  int w_row_bytes;
  int cpg_shift;          // log2(16-byte chunks per scale group)
  int groups_per_row;
  int ksteps;             // K / 128
  TileMap map;
  OutArgs out;
};

// WM x WN waves, each owning TM x TN MFMA tiles of 32 x 32.  G32: one scale per
// 16-byte chunk (group size 32), the two scales of a lane's step come as one
// 4-byte load.
template <int WM, int WN, int TM, int TN, bool G32>
__global__ __launch_bounds__(WM * WN * 64) void gemm_direct_kernel(const DirectArgs a) {
  constexpr int THREADS = WM * WN * 64;
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  constexpr int X_LOADS = BM * 16 / THREADS;  // 16-byte units of the X tile per thread per step
  static_assert(BM * 16 % THREADS == 0, "X tile must divide over the threads");
  constexpr int STAGE_UNITS = BM * DROW_UNITS;
  extern __shared__ u32x4 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave / WN, wn = wave % WN;
  const int lrow = lane & 31, lk = lane >> 5;

  int tm_idx, tn_idx;
  if (!tile_of(a.map, blockIdx.x, tm_idx, tn_idx)) return;  // padding of the tile map (whole workgroup)
  const int m0 = tm_idx * BM, n0 = tn_idx * BN;

  // The lane's weight rows: 64 bytes of a row per step, this lane takes bytes 32*lk .. 32*lk+31.
  const uint8_t* wptr[TN];
  const uint16_t* sptr[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int row = min(n0 + (wn * TN + j) * 32 + lrow, a.n - 1);
    wptr[j] = a.packed + (size_t)row * a.w_row_bytes + lk * 32;
    sptr[j] = a.scales + (size_t)row * a.groups_per_row;
  }

  // Raw loaded values only; nothing is converted at issue time.
  struct BStage {
    u32x4 w[TN][2];
    uint32_t s[TN][2];  // G32: s[j][0] holds both scales; else one 16-bit scale each
  };
  auto load_b = [&](int step, BStage& b) {
    const int st = min(step, a.ksteps - 1);  // past the end: a harmless reload of the last step
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const u32x4* src = (const u32x4*)(wptr[j] + (size_t)st * 64);
      b.w[j][0] = src[0];
      b.w[j][1] = src[1];
      if (G32) {
        b.s[j][0] = *(const uint32_t*)(sptr[j] + st * 4 + lk * 2);
      } else {
        const int ch = st * 4 + lk * 2;
        b.s[j][0] = sptr[j][ch >> a.cpg_shift];
        b.s[j][1] = sptr[j][(ch + 1) >> a.cpg_shift];
      }
    }
  };
  // X goes through registers in two halves (units i < XH, then the rest), each
  // loaded before one half of the step's MFMAs and stored to LDS after it: half
  // the staging registers, and the loads still have a half step to arrive.
  constexpr int XH = X_LOADS / 2;
  static_assert(X_LOADS % 2 == 0, "X tile units per thread must be even");
  u32x4 xr[XH];
  auto load_x = [&](int step, int half) {
    const int k0 = min(step, a.ksteps - 1) * DK;
#pragma unroll
    for (int i = 0; i < XH; ++i) {
      const int u = tid + (half * XH + i) * THREADS;
      const int row = min(m0 + (u >> 4), a.m - 1);
      xr[i] = *(const u32x4*)(a.x + (size_t)row * a.k + k0 + (u & 15) * 8);
    }
  };
  auto store_x = [&](int buf, int half) {
    u32x4* xs = lds + buf * STAGE_UNITS;
#pragma unroll
    for (int i = 0; i < XH; ++i) {
      const int u = tid + (half * XH + i) * THREADS;
      xs[(u >> 4) * DROW_UNITS + (u & 15)] = permute_x_for_int4(xr[i]);
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // One step = 8 MFMA groups kk = 4*c + w.  They are software pipelined by hand:
  // while the MFMAs of group kk run, the A operands of group kk+1 are read from
  // LDS and its B operands dequantised, into the other of two operand sets; the
  // B operands of the NEXT step's first group are prepared during the last
  // group, before the barrier.  An MFMA occupies the matrix pipe for 8 passes and
  // the wave can issue 7 other instructions meanwhile, so written in this order
  // the dequantisation and the LDS reads hide under the MFMAs of the same wave.
  auto dequant = [&](const BStage& b, int kk, half8_t (&bf)[TN]) {
    const int c = kk >> 2, w = kk & 3;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const uint32_t bits = G32 ? (c ? (b.s[j][0] >> 16) : (b.s[j][0] & 0xffffu)) : b.s[j][c];
      const _Float16 sh = __builtin_bit_cast(_Float16, (uint16_t)bits);
      const half2_t s2 = {sh, sh};
      const u32x4 chunk = b.w[j][c];
      const uint32_t word = w == 0 ? chunk.x : (w == 1 ? chunk.y : (w == 2 ? chunk.z : chunk.w));
      half2_t h[4];
      unpack_int4_word(word, h);
      half8_t v;
      const half2_t h0 = h[0] * s2, h1 = h[1] * s2, h2 = h[2] * s2, h3 = h[3] * s2;
      v[0] = h0[0]; v[1] = h0[1]; v[2] = h1[0]; v[3] = h1[1];
      v[4] = h2[0]; v[5] = h2[1]; v[6] = h3[0]; v[7] = h3[1];
      bf[j] = v;
    }
  };
  auto read_a = [&](int buf, int kk, half8_t (&af)[TM]) {
    const u32x4* xs = lds + buf * STAGE_UNITS + (wm * TM * 32 + lrow) * DROW_UNITS + lk * 8 + kk;
#pragma unroll
    for (int i = 0; i < TM; ++i) af[i] = __builtin_bit_cast(half8_t, xs[i * 32 * DROW_UNITS]);
  };
  auto mfmas = [&](const half8_t (&af)[TM], const half8_t (&bf)[TN]) {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
  };

  // Two weight stages ping-pong (no copies, no dynamic indexing); X of step s+1 is
  // loaded to registers while step s computes and goes to the other LDS buffer.
  // Every load is unconditional (clamped past the end).
  BStage b0, b1;
  half8_t afA[TM], afB[TM], bfA[TN], bfB[TN];
  load_x(0, 0);
  load_b(0, b0);
  load_b(1, b1);
  store_x(0, 0);
  load_x(0, 1);
  store_x(0, 1);
  dequant(b0, 0, bfA);
  lds_barrier();
  // The scheduling fences keep the compiler from sinking the X loads to their
  // use (the LDS store), which would expose their latency.
  auto step = [&](int s, BStage& b, const BStage& bnext) {
    const int buf = s & 1;
    load_x(s + 1, 0);
    read_a(buf, 0, afA);
    __builtin_amdgcn_sched_barrier(0);
    read_a(buf, 1, afB); dequant(b, 1, bfB); mfmas(afA, bfA);
    read_a(buf, 2, afA); dequant(b, 2, bfA); mfmas(afB, bfB);
    read_a(buf, 3, afB); dequant(b, 3, bfB); mfmas(afA, bfA);
    read_a(buf, 4, afA); dequant(b, 4, bfA); mfmas(afB, bfB);
    __builtin_amdgcn_sched_barrier(0);
    store_x(buf ^ 1, 0);
    load_x(s + 1, 1);
    __builtin_amdgcn_sched_barrier(0);
    read_a(buf, 5, afB); dequant(b, 5, bfB); mfmas(afA, bfA);
    read_a(buf, 6, afA); dequant(b, 6, bfA); mfmas(afB, bfB);
    read_a(buf, 7, afB); dequant(b, 7, bfB); mfmas(afA, bfA);
    dequant(bnext, 0, bfA); mfmas(afB, bfB);
    __builtin_amdgcn_sched_barrier(0);
    load_b(s + 2, b);
    store_x(buf ^ 1, 1);
    lds_barrier();
  };
  // Whole pairs in the loop and the odd step after it: a step under a branch
  // inside the loop would make the wait counters at the loop head assume that the
  // stage consumed next was refilled one step ago, and stall on it.
  int s = 0;
  for (; s + 1 < a.ksteps; s += 2) {
    step(s, b0, b1);
    step(s + 1, b1, b0);
  }
  if (s < a.ksteps) step(s, b0, b1);

  // Epilogue: one 32-row block of the wave at a time through a private LDS patch
  // (the staging buffers are free after the last barrier).
  float* patch = (float*)lds + wave * (32 * (TN * 32 + 4));
#pragma unroll
  for (int i = 0; i < TM; ++i)
    wave_epilogue<TN>(patch, acc[i], lane, m0 + (wm * TM + i) * 32, n0 + wn * TN * 32, a.out);
}

template <int WM, int WN, int TM, int TN>
int launch_direct_tile(const DirectArgs& a, bool g32, hipStream_t stream) {
  constexpr int BM = WM * TM * 32, BN = WN * TN * 32;
  const void* fn = g32 ? (const void*)gemm_direct_kernel<WM, WN, TM, TN, true>
                       : (const void*)gemm_direct_kernel<WM, WN, TM, TN, false>;
  size_t lds_bytes = (size_t)2 * BM * DROW_UNITS * 16;
  const size_t patch_bytes = (size_t)WM * WN * 32 * (TN * 32 + 4) * sizeof(float);
  if (lds_bytes < patch_bytes) lds_bytes = patch_bytes;
  if (lds_bytes > 64 * 1024)
    TLHIP_CHECK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes));
  DirectArgs b = a;
  int grid = 0;
  b.map = make_tile_map((a.m + BM - 1) / BM, (a.n + BN - 1) / BN, &grid);
  void* args[] = {(void*)&b};
  TLHIP_CHECK_HIP(hipLaunchKernel(fn, dim3(grid), dim3(WM * WN * 64), args, lds_bytes, stream));
  return TLHIP_OK;
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
};

}  // namespace

bool gemm_direct_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  static const char* reasons[] = {
      "not the tiled_direct variant",
      "weights must be int4-grouped",
      "activations must be f16",
      "K must be a multiple of 128",
      "group size must be a multiple of 32",
      "tile (M, N, waves M, waves N) must be one of 256x256 2x4, 256x128 2x4, 128x256 2x4, 256x128 4x2, 128x128 2x2, 256x256 2x2 with tile K 128",
  };
  auto fail = [&](int i) {
    if (why) *why = reasons[i];
    return false;
  };
  if (c.variant != VARIANT_TILED_DIRECT) return fail(0);
  if (p.format != TLHIP_FMT_INT4_GROUPED) return fail(1);
  if (p.x_dtype != TLHIP_F16) return fail(2);
  if (p.k % DK != 0 || p.k == 0) return fail(3);
  if (p.group_size % 32 != 0) return fail(4);
  if (c.p2 != DK) return fail(5);
  for (const auto& t : kDirectTiles)
    if (t.bm == c.p0 && t.bn == c.p1 && t.wm == c.p3 && t.wn == c.p4) return true;
  return fail(5);
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
  a.w_row_bytes = (int)(p.k / 2);
  a.cpg_shift = __builtin_ctz((unsigned)(p.group_size / 32));
  a.groups_per_row = (int)(p.k / p.group_size);
  a.ksteps = (int)(p.k / DK);
  a.out.y = p.y;
  a.out.y_dtype = p.y_dtype;
  a.out.vec_ok = (p.n % 8 == 0) && ((uintptr_t)p.y % 16 == 0);
  a.out.m = (int)p.m;
  a.out.n = (int)p.n;
  a.out.alpha = p.alpha;
  a.out.epi = p.epi;
  const bool g32 = p.group_size == 32;
  int rc;
  if (c.p0 == 256 && c.p1 == 256 && c.p4 == 2) rc = launch_direct_tile<2, 2, 4, 4>(a, g32, stream);
  else if (c.p0 == 256 && c.p1 == 256) rc = launch_direct_tile<2, 4, 4, 2>(a, g32, stream);
  else if (c.p0 == 256 && c.p1 == 128 && c.p3 == 2) rc = launch_direct_tile<2, 4, 4, 1>(a, g32, stream);
  else if (c.p0 == 128 && c.p1 == 256) rc = launch_direct_tile<2, 4, 2, 2>(a, g32, stream);
  else if (c.p0 == 128 && c.p1 == 128) rc = launch_direct_tile<2, 2, 2, 2>(a, g32, stream);
  else rc = launch_direct_tile<4, 2, 2, 2>(a, g32, stream);
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  count_gemm_dispatch();
  return TLHIP_OK;
}

}  // namespace tlhip
