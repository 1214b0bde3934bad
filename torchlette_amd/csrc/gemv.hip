// Decode GEMV / skinny GEMM over packed weights with fused dequant, VALU form.
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
#include "device_utils.h"

namespace tlhip {
namespace {

struct GemvArgs {
  const u32x4* packed;
  const void* scales;
  const void* x;
  void* y;
  int64_t n;
  int k;
  int m;
  int nchunks;           // 16-byte chunks per weight row
  int cpg_shift;         // grouped formats: log2(chunks sharing one scale)
  int groups_per_row;
  int lpr;               // lanes per row
  int kw;                // waves splitting K inside a workgroup
  int slice_chunks;      // chunks of x resident in LDS at a time
  int nslices;
  int nblocks;           // row blocks
  int rows_per_wave;
  int rows_per_wg;
  float alpha;
  float scale_mul;       // 1/127 for INT8_GROUPED, else 1
  int y_dtype;
  DevEpilogue epi;
};

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
// chunk c) lives at unit index (m*NQ + qd)*slice_chunks + c, so the lanes of a
// row group, which hold consecutive c, read consecutive units.
template <int FMT, typename XT, int MT, int R, int U>
__global__ __launch_bounds__(512) void gemv_kernel(const GemvArgs a) {
  using Dot = ChunkDot<FMT, XT>;
  constexpr int NQ = Dot::NQ;
  constexpr bool GROUPED = (FMT != TLHIP_FMT_INT8_ROW);
  extern __shared__ u32x4 lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int kw_idx = wave % a.kw;
  const int rg = wave / a.kw;
  const int sub = lane / a.lpr;
  const int lj = lane - sub * a.lpr;
  const int cstride = a.lpr * a.kw;
  const int cfirst = kw_idx * a.lpr + lj;
  const int x_units_per_row = a.k * (int)sizeof(XT) / 16;  // 16-byte units per activation row
  const u32x4* xg = (const u32x4*)a.x;
  u32x4* partial = lds + (size_t)MT * NQ * a.slice_chunks;  // kw x rows_per_wg x MT floats, if kw > 1

  auto stage = [&](int slice) {
    const int c0 = slice * a.slice_chunks;
    const int cn = min(a.slice_chunks, a.nchunks - c0);
    const int units = cn * NQ;
    for (int m = 0; m < MT; ++m) {
      const int mm = m < a.m ? m : a.m - 1;  // rows beyond m replicate the last row; never stored
      for (int u = tid; u < units; u += blockDim.x) {
        u32x4 v = xg[(size_t)mm * x_units_per_row + (size_t)c0 * NQ + u];
        if (FMT == TLHIP_FMT_INT4_GROUPED && sizeof(XT) == 2) v = permute_x_for_int4(v);
        const int c = u / NQ, qd = u - c * NQ;
        lds[(m * NQ + qd) * a.slice_chunks + c] = v;
      }
    }
  };

  if (a.nslices == 1) {
    stage(0);
    __syncthreads();
  }

  for (int rb = blockIdx.x; rb < a.nblocks; rb += gridDim.x) {
    const int64_t row0 = (int64_t)rb * a.rows_per_wg + rg * a.rows_per_wave + sub * R;
    float acc[R][MT];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[r][m] = 0.f;

    const u32x4* wrow[R];
    const uint16_t* srow[R];
    float row_scale[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t row = min(row0 + r, a.n - 1);  // tail rows recompute the last row; store is masked
      wrow[r] = a.packed + row * a.nchunks;
      if (GROUPED) {
        srow[r] = (const uint16_t*)a.scales + row * a.groups_per_row;
        row_scale[r] = 1.f;
      } else {
        srow[r] = nullptr;
        row_scale[r] = ((const float*)a.scales)[row];
      }
    }

    for (int slice = 0; slice < a.nslices; ++slice) {
      if (a.nslices > 1) {
        __syncthreads();
        stage(slice);
        __syncthreads();
      }
      const int c_begin = slice * a.slice_chunks;
      const int c_end = min(c_begin + a.slice_chunks, a.nchunks);
      for (int cb = c_begin + cfirst; cb < c_end; cb += cstride * U) {
        u32x4 wv[U][R];
        float sv[U][R];
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int c = cb + u * cstride;
          if (c < c_end) {
#pragma unroll
            for (int r = 0; r < R; ++r) {
              wv[u][r] = __builtin_nontemporal_load(wrow[r] + c);
              if (GROUPED) sv[u][r] = half_bits_to_float(srow[r][c >> a.cpg_shift]);
            }
          }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
          const int c = cb + u * cstride;
          if (c < c_end) {
            const int cl = c - c_begin;
            u32x4 xv[MT][NQ];
#pragma unroll
            for (int m = 0; m < MT; ++m)
#pragma unroll
              for (int qd = 0; qd < NQ; ++qd) xv[m][qd] = lds[(m * NQ + qd) * a.slice_chunks + cl];
#pragma unroll
            for (int r = 0; r < R; ++r) {
              Dot d;
              d.unpack(wv[u][r]);
#pragma unroll
              for (int m = 0; m < MT; ++m) {
                const float part = d.dot(xv[m]);
                if (GROUPED) acc[r][m] = fmaf(sv[u][r], part, acc[r][m]);
                else acc[r][m] += part;
              }
            }
          }
        }
      }
    }

    // lanes of a row group -> one sum (all lanes of the group hold it)
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[r][m] = group_sum(acc[r][m], a.lpr);

    if (a.kw > 1) {
      // split-K combine through LDS: partial[kw][row in wg][m]
      float* pf = (float*)partial;
      __syncthreads();
      if (lj == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < MT; ++m)
            pf[((kw_idx * a.rows_per_wg) + rg * a.rows_per_wave + sub * R + r) * MT + m] = acc[r][m];
      }
      __syncthreads();
      if (kw_idx == 0 && lj == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r)
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            float s = 0.f;
            for (int w = 0; w < a.kw; ++w)
              s += pf[((w * a.rows_per_wg) + rg * a.rows_per_wave + sub * R + r) * MT + m];
            acc[r][m] = s;
          }
      }
    }

    if (kw_idx == 0 && lj == 0) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int64_t row = row0 + r;
        if (row < a.n) {
#pragma unroll
          for (int m = 0; m < MT; ++m) {
            if (m < a.m) {
              float v = acc[r][m] * (row_scale[r] * a.scale_mul) * a.alpha;
              v = apply_epilogue(a.epi, v, row);
              store_out(a.y, a.y_dtype, (int64_t)m * a.n + row, v);
            }
          }
        }
      }
    }
  }
}

constexpr int kLdsBudget = 64 * 1024;

template <int FMT, typename XT, int MT, int R>
int launch_t(const GemvArgs& a, int threads, int grid, size_t lds_bytes, hipStream_t stream) {
  hipLaunchKernelGGL((gemv_kernel<FMT, XT, MT, R, 2>), dim3(grid), dim3(threads), lds_bytes, stream, a);
  return TLHIP_OK;
}

template <int FMT, typename XT, int MT>
int launch_r(int r, const GemvArgs& a, int threads, int grid, size_t lds_bytes, hipStream_t stream) {
  switch (r) {
    case 1: return launch_t<FMT, XT, MT, 1>(a, threads, grid, lds_bytes, stream);
    case 2: return launch_t<FMT, XT, MT, 2>(a, threads, grid, lds_bytes, stream);
    case 4: return launch_t<FMT, XT, MT, 4>(a, threads, grid, lds_bytes, stream);
  }
  return set_error(TLHIP_ERR_INVALID, "gemv: rows per lane group must be 1, 2 or 4 (got %d)", r);
}

template <int FMT, typename XT>
int launch_m(int mt, int r, const GemvArgs& a, int threads, int grid, size_t lds_bytes, hipStream_t stream) {
  switch (mt) {
    case 1: return launch_r<FMT, XT, 1>(r, a, threads, grid, lds_bytes, stream);
    case 2: return launch_r<FMT, XT, 2>(r, a, threads, grid, lds_bytes, stream);
    case 4: return launch_r<FMT, XT, 4>(r, a, threads, grid, lds_bytes, stream);
  }
  return set_error(TLHIP_ERR_INVALID, "gemv: internal M tile %d", mt);
}

template <int FMT>
int launch_x(int x_dtype, int mt, int r, const GemvArgs& a, int threads, int grid, size_t lds_bytes,
             hipStream_t stream) {
  if (x_dtype == TLHIP_F16) return launch_m<FMT, _Float16>(mt, r, a, threads, grid, lds_bytes, stream);
  return launch_m<FMT, float>(mt, r, a, threads, grid, lds_bytes, stream);
}

int chunk_weights(int format) { return format == TLHIP_FMT_INT4_GROUPED ? 32 : 16; }

}  // namespace

bool gemv_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  static const char* reasons[] = {
      "not the gemv variant",
      "lanes per row must be 16, 32 or 64",
      "rows per lane group must be 1, 2 or 4",
      "waves per workgroup must be 1..8",
      "K-split waves must divide waves per workgroup",
      "K must be a whole number of 16-byte chunks (K % 32 for int4, K % 16 for int8)",
      "group size must be a multiple of the chunk (32 for int4, 16 for int8)",
      "M above 16",
  };
  auto fail = [&](int i) {
    if (why) *why = reasons[i];
    return false;
  };
  if (c.variant != VARIANT_GEMV) return fail(0);
  if (c.p0 != 16 && c.p0 != 32 && c.p0 != 64) return fail(1);
  if (c.p1 != 1 && c.p1 != 2 && c.p1 != 4) return fail(2);
  if (c.p2 < 1 || c.p2 > 8) return fail(3);
  if (c.p3 < 1 || c.p2 % c.p3 != 0) return fail(4);
  const int cw = chunk_weights(p.format);
  if (p.k % cw != 0) return fail(5);
  if (p.format != TLHIP_FMT_INT8_ROW && p.group_size % cw != 0) return fail(6);
  if (p.m > 16) return fail(7);
  return true;
}

// One launch handles at most 4 activation rows; larger M is issued as passes of
// 4 rows (each pass streams the weights again — the MFMA variant avoids that).
int launch_gemv(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_config_applicable(p, c, &why)) return set_error(TLHIP_ERR_INVALID, "gemv: config not applicable: %s", why);
  if (p.n == 0 || p.m == 0) return TLHIP_OK;
  const int cw = chunk_weights(p.format);
  const int xbytes = p.x_dtype == TLHIP_F16 ? 2 : 4;
  const int ybytes = p.y_dtype == TLHIP_F16 ? 2 : 4;

  for (int64_t m0 = 0; m0 < p.m; m0 += 4) {
    const int mrows = (int)(p.m - m0 < 4 ? p.m - m0 : 4);
    const int mt = mrows == 1 ? 1 : (mrows == 2 ? 2 : 4);
    GemvArgs a;
    a.packed = (const u32x4*)p.packed;
    a.scales = p.scales;
    a.x = (const char*)p.x + m0 * p.k * xbytes;
    a.y = (char*)p.y + m0 * p.n * ybytes;
    a.n = p.n;
    a.k = (int)p.k;
    a.m = mrows;
    a.nchunks = (int)(p.k / cw);
    a.cpg_shift = p.format == TLHIP_FMT_INT8_ROW ? 0 : __builtin_ctz((unsigned)(p.group_size / cw));
    a.groups_per_row = p.format == TLHIP_FMT_INT8_ROW ? 0 : (int)(p.k / p.group_size);
    a.lpr = c.p0;
    a.kw = c.p3;
    const int r = c.p1, waves = c.p2;
    a.rows_per_wave = (64 / a.lpr) * r;
    a.rows_per_wg = (waves / a.kw) * a.rows_per_wave;
    a.nblocks = (int)((p.n + a.rows_per_wg - 1) / a.rows_per_wg);
    a.alpha = p.alpha;
    a.scale_mul = p.format == TLHIP_FMT_INT8_GROUPED ? (1.0f / 127.0f) : 1.0f;
    a.y_dtype = p.y_dtype;
    a.epi = p.epi;
    // LDS: staged x (mt rows x slice) + split-K partials
    const int chunk_x_bytes = cw * xbytes;
    const size_t partial_bytes = a.kw > 1 ? (size_t)a.kw * a.rows_per_wg * mt * sizeof(float) : 0;
    int max_slice_chunks = (int)((kLdsBudget - partial_bytes) / ((size_t)mt * chunk_x_bytes));
    if (max_slice_chunks >= a.nchunks) {
      a.slice_chunks = a.nchunks;
      a.nslices = 1;
    } else {
      // whole multiples of the chunk stride so every slice starts on the same lane phase
      const int cstride = a.lpr * a.kw;
      int sc = max_slice_chunks / cstride * cstride;
      if (sc <= 0) return set_error(TLHIP_ERR_INVALID, "gemv: K slice does not fit LDS for this configuration");
      a.slice_chunks = sc;
      a.nslices = (a.nchunks + sc - 1) / sc;
    }
    const size_t lds_bytes = (size_t)mt * chunk_x_bytes * a.slice_chunks + partial_bytes;
    const int threads = waves * 64;
    const int cus = device_cu_count();
    // resident workgroups per CU: bounded by 2048 lanes and by LDS
    int per_cu = 2048 / threads;
    const int by_lds = (int)((160 * 1024) / (lds_bytes ? lds_bytes : 1));
    if (by_lds < per_cu) per_cu = by_lds < 1 ? 1 : by_lds;
    if (per_cu < 1) per_cu = 1;
    int grid = a.nblocks < cus * per_cu ? a.nblocks : cus * per_cu;
    if (grid < 1) grid = 1;
    int rc;
    switch (p.format) {
      case TLHIP_FMT_INT4_GROUPED:
        rc = launch_x<TLHIP_FMT_INT4_GROUPED>(p.x_dtype, mt, r, a, threads, grid, lds_bytes, stream);
        break;
      case TLHIP_FMT_INT8_GROUPED:
        rc = launch_x<TLHIP_FMT_INT8_GROUPED>(p.x_dtype, mt, r, a, threads, grid, lds_bytes, stream);
        break;
      default:
        rc = launch_x<TLHIP_FMT_INT8_ROW>(p.x_dtype, mt, r, a, threads, grid, lds_bytes, stream);
        break;
    }
    if (rc) return rc;
    TLHIP_CHECK_HIP(hipGetLastError());
  }
  count_gemv_dispatch();
  return TLHIP_OK;
}

}  // namespace tlhip
