// Prefill GEMM over packed weights: Y[M,N] = epilogue(alpha * X[M,K] * W[N,K]^T)
// with the dequantisation fused into the LDS stage.  Stands in for the
// reference's M > 1 route — an explicit dequant to an f32 [N,K] buffer followed
// by the stock tiled matmul (src/backend/webgpu/ops/matmul-ops.ts:163-181;
// src/schedule/matmul-skeleton.ts:738-966) — without ever materialising the
// dequantised weight in HBM.
//
// MFMA-bound (f16 inputs, f32 accumulate).  One workgroup of 4 waves (2 x 2)
// computes a BM x BN tile of Y with v_mfma_f32_32x32x16_f16; a wave owns a
// (BM/2) x (BN/2) sub-tile, i.e. (BM/64) x (BN/64) MFMA tiles of 16
// accumulators each.  Per K step of 64:
//   * global -> registers: the X tile (f16, 16 bytes per lane per load) and the
//     packed W tile (16 bytes = 32 int4 or 16 int8 weights, plus the group
//     scale), three or four steps ahead, in a ring of register stages;
//   * registers -> LDS: the weights are unpacked to exact integers in f16 and
//     multiplied by their scale (packed f16 multiply, one rounding to f16 per
//     weight), then written k-contiguous; X is written as is (for int4, with
//     the same within-8 k order the unpack produces);
//   * LDS -> MFMA operands: rows are padded to 144 bytes so that the 32 lanes of
//     an operand read hit 16 different 16-byte bank groups.
// LDS is double buffered (one barrier per K step, and the barrier waits for LDS
// traffic only, not for the global loads in flight).
// Epilogue: acc*alpha -> ops in order (bias indexed by n, unary) -> cast, the
// order of applyBlockEpilogue (matmul-skeleton.ts:916-966).
#include <cstring>

#include "gemm_common.h"

namespace tlhip {
namespace {

constexpr int BK = 64;                 // k per step
constexpr int ROW_BYTES = BK * 2 + 16; // padded LDS row: 144 bytes = 9 units
constexpr int ROW_UNITS = ROW_BYTES / 16;

struct GemmArgs {
  const uint8_t* packed;  // bytes; row stride row_bytes
  const void* scales;
  const _Float16* x;
  int m, n, k;
  int w_row_bytes;        // K/2 (int4) or K (int8)
  int cpg_shift;          // log2(16-byte chunks per scale group)
  int groups_per_row;
  int ksteps;
  TileMap map;
  OutArgs out;
  int ksplit;             // workgroups that share a tile, each walking ksteps / ksplit steps of K (1 = none)
  float* workspace;       // ksplit > 1: the slices' partial sums, [slice][M][N] f32
};

// Unpack one 16-byte chunk to f16 values already multiplied by the scale.
// int4: 32 weights -> 4 units (64 bytes) in the (0,4,1,5,2,6,3,7) order per word.
// int8: 16 weights -> 2 units (32 bytes), natural order.
template <int FMT>
struct WChunk;

template <>
struct WChunk<TLHIP_FMT_INT4_GROUPED> {
  static constexpr int WEIGHTS = 32;
  static constexpr int UNITS = 4;
  __device__ static __forceinline__ void dequant(const u32x4& w, float scale, u32x4 (&out)[UNITS]) {
    const _Float16 sh = (_Float16)scale;  // the scale is an f16 value: exact
    const half2_t s2 = {sh, sh};
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half2_t h[4];
      unpack_int4_word(words[i], h);
      u32x4 o;
      o.x = __builtin_bit_cast(uint32_t, h[0] * s2);
      o.y = __builtin_bit_cast(uint32_t, h[1] * s2);
      o.z = __builtin_bit_cast(uint32_t, h[2] * s2);
      o.w = __builtin_bit_cast(uint32_t, h[3] * s2);
      out[i] = o;
    }
  }
};

// int8 with an f16 scale per group: the integer (exact in f16) times the scale as it is
// stored, one rounding to f16 per weight; the format's 1/127 rides on alpha.
template <>
struct WChunk<TLHIP_FMT_INT8_GROUPED> {
  static constexpr int WEIGHTS = 16;
  static constexpr int UNITS = 2;
  __device__ static __forceinline__ void dequant(const u32x4& w, float scale, u32x4 (&out)[UNITS]) {
    const _Float16 sh = (_Float16)scale;  // the scale is an f16 value: exact
    const half2_t s2 = {sh, sh};
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
    uint32_t packed[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half2_t h[2];
      unpack_int8_word(words[i], h);
      packed[2 * i] = __builtin_bit_cast(uint32_t, h[0] * s2);
      packed[2 * i + 1] = __builtin_bit_cast(uint32_t, h[1] * s2);
    }
    out[0] = (u32x4){packed[0], packed[1], packed[2], packed[3]};
    out[1] = (u32x4){packed[4], packed[5], packed[6], packed[7]};
  }
};
// int8 with one f32 scale per row: the bare integers go to the matrix cores (exact in f16)
// and the row's scale multiplies the f32 sums in the epilogue, as a factor per output
// column: no rounding of q * s to f16, and no scale that f16 could not hold.
template <>
struct WChunk<TLHIP_FMT_INT8_ROW> {
  static constexpr int WEIGHTS = 16;
  static constexpr int UNITS = 2;
  __device__ static __forceinline__ void dequant(const u32x4& w, float, u32x4 (&out)[UNITS]) {
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
    uint32_t packed[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      half2_t h[2];
      unpack_int8_word(words[i], h);
      packed[2 * i] = __builtin_bit_cast(uint32_t, h[0]);
      packed[2 * i + 1] = __builtin_bit_cast(uint32_t, h[1]);
    }
    out[0] = (u32x4){packed[0], packed[1], packed[2], packed[3]};
    out[1] = (u32x4){packed[4], packed[5], packed[6], packed[7]};
  }
};

// SPLIT: the instances that take K slices across workgroups (the 64- and 128-row tiles
// with 128 columns, the ones a launch of few tiles uses); the others compile as without.
template <int FMT, int BM, int BN, bool SPLIT>
__global__ __launch_bounds__(256) void gemm_prefill_kernel(const GemmArgs a) {
  using WC = WChunk<FMT>;
  constexpr bool GROUPED = (FMT != TLHIP_FMT_INT8_ROW);
  constexpr int TM = BM / 64, TN = BN / 64;        // MFMA tiles per wave
  constexpr int X_LOADS = BM * 8 / 256;            // 16-byte units of the X tile per thread
  constexpr int W_CHUNKS_PER_ROW = BK / WC::WEIGHTS;
  constexpr int W_LOADS = BN * W_CHUNKS_PER_ROW / 256;
  constexpr int STAGE_UNITS = (BM + BN) * ROW_UNITS;
  extern __shared__ u32x4 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // K split across workgroups, as in gemm_direct.hip: the ksplit workgroups of consecutive
  // ids take the slices of one tile and leave their partial sums in the workspace.
  const int slice = SPLIT ? (int)(blockIdx.x % (unsigned)a.ksplit) : 0;
  const int tile_id = SPLIT ? (int)(blockIdx.x / (unsigned)a.ksplit) : (int)blockIdx.x;
  const int nsteps = SPLIT ? a.ksteps / a.ksplit : a.ksteps;
  const int step0 = slice * nsteps;
  int tm_idx, tn_idx;
  if (!tile_of(a.map, tile_id, tm_idx, tn_idx)) return;  // padding of the tile map (whole workgroup)
  const int m0 = tm_idx * BM, n0 = tn_idx * BN;

  // ---- global -> register staging -------------------------------------
  // A ring of D register stages: the tiles of K step j live in stage j % D.
  // At step ks the loads for step ks+D are issued (into the stage that held
  // step ks, already in LDS), the tiles of step ks+1 go from registers to the
  // other LDS buffer, and the MFMAs run on step ks: every global load has D-1
  // full steps to arrive.  All loads are unconditional (clamped at the end).
  // (the int8 formats hold twice the packed weights per stage: three stages from 384 rows
  // of tiles on, or the largest instances run out of registers)
  constexpr int D = ((BM + BN) >= 512 || (FMT != TLHIP_FMT_INT4_GROUPED && (BM + BN) >= 384)) ? 3 : 4;
  u32x4 xr[D][X_LOADS];
  u32x4 wr[D][W_LOADS];
  uint32_t sr[D][W_LOADS];  // raw scale bits (f16) or f32 bits (int8-row)

  auto load_tiles = [&](int kstep, u32x4 (&xs)[X_LOADS], u32x4 (&ws)[W_LOADS], uint32_t (&ss)[W_LOADS]) {
    const int k0 = (step0 + min(kstep, nsteps - 1)) * BK;
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) {
      const int u = tid + i * 256;
      const int row = min(m0 + (u >> 3), a.m - 1);
      xs[i] = *(const u32x4*)(a.x + (size_t)row * a.k + k0 + (u & 7) * 8);
    }
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      const int u = tid + i * 256;
      const int r = u / W_CHUNKS_PER_ROW, c = u - r * W_CHUNKS_PER_ROW;
      const int row = min(n0 + r, a.n - 1);
      const int chunk = k0 / WC::WEIGHTS + c;
      ws[i] = *(const u32x4*)(a.packed + (size_t)row * a.w_row_bytes + (size_t)chunk * 16);
      if (GROUPED) ss[i] = ((const uint16_t*)a.scales)[(size_t)row * a.groups_per_row + (chunk >> a.cpg_shift)];
      else ss[i] = 0;  // int8-row: the row scales are the epilogue's
    }
  };

  auto store_tiles = [&](int buf, const u32x4 (&xv)[X_LOADS], const u32x4 (&wv)[W_LOADS],
                         const uint32_t (&sv)[W_LOADS]) {
    u32x4* xs = lds + buf * STAGE_UNITS;
    u32x4* ws = xs + BM * ROW_UNITS;
#pragma unroll
    for (int i = 0; i < X_LOADS; ++i) {
      const int u = tid + i * 256;
      u32x4 v = xv[i];
      if (FMT == TLHIP_FMT_INT4_GROUPED) v = permute_x_for_int4(v);
      xs[(u >> 3) * ROW_UNITS + (u & 7)] = v;
    }
#pragma unroll
    for (int i = 0; i < W_LOADS; ++i) {
      const int u = tid + i * 256;
      const int r = u / W_CHUNKS_PER_ROW, c = u - r * W_CHUNKS_PER_ROW;
      const float s = GROUPED ? half_bits_to_float(sv[i]) : 1.f;  // int8-row: the row scales are the epilogue's
      u32x4 out[WC::UNITS];
      WC::dequant(wv[i], s, out);
#pragma unroll
      for (int j = 0; j < WC::UNITS; ++j) ws[r * ROW_UNITS + c * WC::UNITS + j] = out[j];
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

#pragma unroll
  for (int s = 0; s < D; ++s) load_tiles(s, xr[s], wr[s], sr[s]);
  store_tiles(0, xr[0], wr[0], sr[0]);
  lds_barrier();

  const int lrow = lane & 31, lk = lane >> 5;
  for (int ks0 = 0; ks0 < nsteps; ks0 += D) {
#pragma unroll
    for (int s = 0; s < D; ++s) {
      const int ks = ks0 + s;
      if (ks < nsteps) {  // uniform
        const int buf = ks & 1;
        // stage s held step ks (already in LDS): refill it with step ks + D
        load_tiles(ks + D, xr[s], wr[s], sr[s]);
        const u32x4* xs = lds + buf * STAGE_UNITS;
        const u32x4* ws = xs + BM * ROW_UNITS;
#pragma unroll
        for (int kk = 0; kk < BK / 16; ++kk) {
          half8_t af[TM], bf[TN];
#pragma unroll
          for (int i = 0; i < TM; ++i)
            af[i] = __builtin_bit_cast(half8_t, xs[(wm * (BM / 2) + i * 32 + lrow) * ROW_UNITS + kk * 2 + lk]);
#pragma unroll
          for (int j = 0; j < TN; ++j)
            bf[j] = __builtin_bit_cast(half8_t, ws[(wn * (BN / 2) + j * 32 + lrow) * ROW_UNITS + kk * 2 + lk]);
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }
        // step ks + 1 (stage s+1) -> the other LDS buffer; harmless past the end
        store_tiles(buf ^ 1, xr[(s + 1) % D], wr[(s + 1) % D], sr[(s + 1) % D]);
        lds_barrier();
      }
    }
  }

  // ---- epilogue -----------------------------------------------------------
  // One 32-row block of the wave at a time through a private LDS patch (the
  // staging buffers are free now); see wave_epilogue.  Applying the epilogue
  // straight from the accumulator registers would need 16 x TM x TN inlined
  // copies of it; the compiler then stops unrolling and the accumulators fall
  // into scratch memory.
  float* patch = (float*)lds + wave * (32 * (TN * 32 + 4));
  // a K slice leaves its bare partial sums, f32, row-major, in this slice's M x N plane of
  // the workspace; the reduce launch adds the planes in slice order and runs the epilogue
  float* const plane = SPLIT ? a.workspace + (size_t)slice * a.m * a.n : nullptr;
#pragma unroll
  for (int i = 0; i < TM; ++i)
    wave_epilogue<TN, SPLIT, FMT == TLHIP_FMT_INT8_ROW>(patch, acc[i], lane, m0 + wm * (BM / 2) + i * 32, n0 + wn * (BN / 2),
                                                         a.out, plane);
}

template <int FMT, int BM, int BN>
int launch_tile(const GemmArgs& a, hipStream_t stream) {
  const void* fn = (const void*)gemm_prefill_kernel<FMT, BM, BN, false>;
  if constexpr (BN == 128 && BM <= 128) {
    if (a.ksplit > 1) fn = (const void*)gemm_prefill_kernel<FMT, BM, BN, true>;
  } else {
    if (a.ksplit > 1) return set_error(TLHIP_ERR_INVALID, "gemm: K slices across workgroups take the 64x128 and 128x128 tiles");
  }
  size_t lds_bytes = (size_t)2 * (BM + BN) * ROW_BYTES;
  const size_t patch_bytes = (size_t)4 * 32 * (BN / 64 * 32 + 4) * sizeof(float);
  if (lds_bytes < patch_bytes) lds_bytes = patch_bytes;
  GemmArgs b = a;
  int grid = 0;
  b.map = make_tile_map((a.m + BM - 1) / BM, (a.n + BN - 1) / BN, TileCost{BM * 2, FMT == TLHIP_FMT_INT4_GROUPED ? BN / 2 : BN}, &grid);
  void* args[] = {(void*)&b};
  return launch_kernel(fn, dim3(grid * (a.ksplit > 1 ? a.ksplit : 1)), dim3(256), args, lds_bytes, stream);
}

template <int FMT>
int launch_fmt(int bm, int bn, const GemmArgs& a, hipStream_t stream) {
  if constexpr (FMT == TLHIP_FMT_INT4_GROUPED) {
    if (bm == 256 && bn == 256) return launch_tile<FMT, 256, 256>(a, stream);
  }
  if (bm == 128 && bn == 256) return launch_tile<FMT, 128, 256>(a, stream);
  if (bm == 256 && bn == 128) return launch_tile<FMT, 256, 128>(a, stream);
  if (bm == 128 && bn == 128) return launch_tile<FMT, 128, 128>(a, stream);
  if (bm == 64 && bn == 128) return launch_tile<FMT, 64, 128>(a, stream);
  return set_error(TLHIP_ERR_INVALID, "gemm: tile %dx%d is not built", bm, bn);
}

}  // namespace

bool gemm_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  static const char* reasons[] = {
      "not the tiled variant",
      "activations must be f16",
      "K must be a multiple of 64",
      "group size must be a multiple of 32 (int4) or 16 (int8)",
      "tile must be one of 256x256 (int4 only), 128x256, 256x128, 128x128, 64x128 with tile K 64 and 2x2 waves",
      "K split across workgroups (p5) must be 0, 1 or a power of two up to 16 that divides K / 64, on the 64x128 or "
      "128x128 tile, with the slices' partial sums (p5 x M x N, f32) inside the library's workspace",
  };
  auto fail = [&](int i) {
    if (why) *why = reasons[i];
    return false;
  };
  if (c.variant != VARIANT_TILED) return fail(0);
  if (p.x_dtype != TLHIP_F16) return fail(1);
  if (p.k % 64 != 0 || p.k == 0) return fail(2);
  if (p.format == TLHIP_FMT_INT4_GROUPED && p.group_size % 32 != 0) return fail(3);
  if (p.format == TLHIP_FMT_INT8_GROUPED && p.group_size % 16 != 0) return fail(3);
  const int bm = c.p0, bn = c.p1;
  const bool ok = (bm == 256 && bn == 256) || (bm == 128 && bn == 256) || (bm == 256 && bn == 128) ||
                  (bm == 128 && bn == 128) || (bm == 64 && bn == 128);
  if (!ok || c.p2 != 64 || c.p3 != 2 || c.p4 != 2) return fail(4);
  // the int8 dequantisation needs more registers: its 256 x 256 instance would spill
  if (bm == 256 && bn == 256 && p.format != TLHIP_FMT_INT4_GROUPED) return fail(4);
  const int ks = c.p5 < 1 ? 1 : c.p5;
  if (ks > 1 && (ks > 16 || (ks & (ks - 1)) != 0 || (p.k / BK) % ks != 0 || bn != 128 || bm > 128 ||
                 (size_t)p.m * (size_t)p.n * ks > kSplitWorkspaceFloats))
    return fail(5);
  return true;
}

int launch_gemm(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemm_config_applicable(p, c, &why)) return set_error(TLHIP_ERR_INVALID, "gemm: config not applicable: %s", why);
  if (p.m == 0 || p.n == 0) return TLHIP_OK;
  const bool int4 = p.format == TLHIP_FMT_INT4_GROUPED;
  const int cw = int4 ? 32 : 16;
  GemmArgs a;
  a.packed = (const uint8_t*)p.packed;
  a.scales = p.scales;
  a.x = (const _Float16*)p.x;
  a.m = (int)p.m;
  a.n = (int)p.n;
  a.k = (int)p.k;
  a.w_row_bytes = (int)(int4 ? p.k / 2 : p.k);
  a.cpg_shift = p.format == TLHIP_FMT_INT8_ROW ? 0 : __builtin_ctz((unsigned)(p.group_size / cw));
  a.groups_per_row = p.format == TLHIP_FMT_INT8_ROW ? 0 : (int)(p.k / p.group_size);
  a.ksteps = (int)(p.k / BK);
  a.ksplit = c.p5 < 1 ? 1 : c.p5;
  a.workspace = nullptr;
  if (a.ksplit > 1) {
    int* counters = nullptr;  // the slices are combined by a second launch, not by arrival
    const int rc = split_workspace(stream, &a.workspace, &counters);
    if (rc) return rc;
  }
  a.out.y = p.y;
  a.out.y_dtype = p.y_dtype;
  a.out.vec_ok = (p.n % 8 == 0) && ((uintptr_t)p.y % 16 == 0);
  a.out.m = (int)p.m;
  a.out.n = (int)p.n;
  // the grouped int8 format's 1/127 (quantize.ts: q = round(w / absmax * 127)) rides on alpha
  a.out.alpha = p.format == TLHIP_FMT_INT8_GROUPED ? p.alpha * (1.0f / 127.0f) : p.alpha;
  a.out.epi = p.epi;
  a.out.col_scale = p.format == TLHIP_FMT_INT8_ROW ? (const float*)p.scales : nullptr;
  int rc;
  switch (p.format) {
    case TLHIP_FMT_INT4_GROUPED: rc = launch_fmt<TLHIP_FMT_INT4_GROUPED>(c.p0, c.p1, a, stream); break;
    case TLHIP_FMT_INT8_GROUPED: rc = launch_fmt<TLHIP_FMT_INT8_GROUPED>(c.p0, c.p1, a, stream); break;
    default: rc = launch_fmt<TLHIP_FMT_INT8_ROW>(c.p0, c.p1, a, stream); break;
  }
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  if (a.ksplit > 1) {
    rc = launch_k_slice_reduce(a.ksplit, a.workspace, a.out, stream);
    if (rc) return rc;
  }
  count_gemm_dispatch();
  return TLHIP_OK;
}

// Every instance launch_gemm can reach, in prepare mode (see launch_kernel).
int prepare_gemm_kernels() {
  GemmArgs a;
  memset(&a, 0, sizeof a);
  a.m = a.n = 1;
  a.ksplit = 1;
  static const int tiles[][2] = {{256, 256}, {128, 256}, {256, 128}, {128, 128}, {64, 128}};
  for (auto& t : tiles) {
    int rc = launch_fmt<TLHIP_FMT_INT4_GROUPED>(t[0], t[1], a, nullptr);
    if (!rc && t[0] * t[1] != 256 * 256) rc = launch_fmt<TLHIP_FMT_INT8_GROUPED>(t[0], t[1], a, nullptr);
    if (!rc && t[0] * t[1] != 256 * 256) rc = launch_fmt<TLHIP_FMT_INT8_ROW>(t[0], t[1], a, nullptr);
    if (!rc && t[1] == 128 && t[0] <= 128) {  // the K-sliced instances of these tiles
      a.ksplit = 2;
      rc = launch_fmt<TLHIP_FMT_INT4_GROUPED>(t[0], t[1], a, nullptr);
      if (!rc) rc = launch_fmt<TLHIP_FMT_INT8_GROUPED>(t[0], t[1], a, nullptr);
      if (!rc) rc = launch_fmt<TLHIP_FMT_INT8_ROW>(t[0], t[1], a, nullptr);
      a.ksplit = 1;
    }
    if (rc) return rc;
  }
  return TLHIP_OK;
}

}  // namespace tlhip
