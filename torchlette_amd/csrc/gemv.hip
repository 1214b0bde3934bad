// Host side of the VALU decode GEMV (stands in for dispatchQuantizedGemvNT,
// src/backend/webgpu/matmul/dispatch.ts:875-931): configuration checks, launch
// geometry, the single and the grouped launch.  The kernel is in gemv_kernel.h and
// is instantiated per weight format in gemv_int4.hip, gemv_int8_grouped.hip and
// gemv_int8_row.hip.
#include <cstring>

#include "gemv_args.h"

namespace tlhip {

namespace {
constexpr int kLdsBudget = 128 * 1024;
int chunk_weights(int format) { return format == TLHIP_FMT_INT4_GROUPED ? 32 : 16; }
}  // namespace

bool gemv_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  static const char* reasons[] = {
      "not the gemv variant",
      "lanes per row must be 16, 32 or 64",
      "rows per lane group must be 1, 2 or 4",
      "waves per workgroup must be 1..8",
      "K-split waves must be 1, 2, 4 or 8 and divide waves per workgroup",
      "K must be a whole number of 16-byte chunks (K % 32 for int4, K % 16 for int8)",
      "group size must be a multiple of the chunk (32 for int4, 16 for int8)",
      "M above 16",
      "chunks in flight must be 2, 4 or 8 with rows*chunks <= 8",
      "the 4x4x4 matrix-core form (p5 = 1) is built for int4 weights, f16 activations, M <= 4, 16 lanes per row, one row per lane group",
      "the activation rows of one pass (K x 2 or 4 bytes each; four rows in the 4x4x4 form) do not fit LDS",
  };
  auto fail = [&](int i) {
    if (why) *why = reasons[i];
    return false;
  };
  if (c.variant != VARIANT_GEMV) return fail(0);
  if (c.p0 != 16 && c.p0 != 32 && c.p0 != 64) return fail(1);
  if (c.p1 != 1 && c.p1 != 2 && c.p1 != 4) return fail(2);
  if (c.p2 < 1 || c.p2 > 8) return fail(3);
  if (c.p3 < 1 || (c.p3 & (c.p3 - 1)) != 0 || c.p2 % c.p3 != 0) return fail(4);
  const int cw = chunk_weights(p.format);
  if (p.k % cw != 0) return fail(5);
  if (p.format != TLHIP_FMT_INT8_ROW && p.group_size % cw != 0) return fail(6);
  if (p.m > 16) return fail(7);
  const int u = c.p4 == 0 ? 2 : c.p4;
  if ((u != 2 && u != 4 && u != 8) || u * c.p1 > 8) return fail(8);
  if (c.p5 != 0 && (c.p5 != 1 || p.format != TLHIP_FMT_INT4_GROUPED || p.x_dtype != TLHIP_F16 || p.m > 4 || c.p0 != 16 ||
                    c.p1 != 1))
    return fail(9);
  // LDS: one activation row must fit next to the partials (more rows per pass only if they
  // fit: see launch_gemv); the 4x4x4 form always stages four
  const size_t xbytes = p.x_dtype == TLHIP_F16 ? 2 : 4;
  const size_t rows = c.p5 == 1 ? 4 : 1;
  if (rows * (size_t)p.k * xbytes + 16 * 1024 > (size_t)kLdsBudget) return fail(10);
  return true;
}

// Kernel arguments and launch geometry of one pass (rows m0 .. m0+mrows of x).
static void fill_args(const Problem& p, const tlhip_kernel_config_t& c, int64_t m0, int mrows, GemvArgs& a, int& mt,
                      int& threads, int& grid, size_t& lds_bytes) {
  const int cw = chunk_weights(p.format);
  const int xbytes = p.x_dtype == TLHIP_F16 ? 2 : 4;
  const int ybytes = p.y_dtype == TLHIP_F16 ? 2 : 4;
  mt = c.p5 == 1 ? 4 : (mrows == 1 ? 1 : (mrows == 2 ? 2 : 4));
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
  a.lpr_shift = __builtin_ctz((unsigned)c.p0);
  a.kw = c.p3;
  a.kw_shift = __builtin_ctz((unsigned)c.p3);
  const int r = c.p1, waves = c.p2, unroll = c.p4 == 0 ? 2 : c.p4;
  a.nsteps = (a.nchunks + a.lpr * a.kw * unroll - 1) / (a.lpr * a.kw * unroll);
  a.rows_per_wave = (64 / a.lpr) * r;
  a.rows_per_wg = (waves / a.kw) * a.rows_per_wave;
  a.nblocks = (int)((p.n + a.rows_per_wg - 1) / a.rows_per_wg);
  a.alpha = p.alpha;
  a.scale_mul = p.format == TLHIP_FMT_INT8_GROUPED ? (1.0f / 127.0f) : 1.0f;
  a.y_dtype = p.y_dtype;
  a.epi = epilogue_from_row(p.epi, m0, p.n);  // this pass starts at row m0, like y
  a.pro = p.pro;
  if (a.pro.kind == TLHIP_PRO_GATED_MUL) a.pro.operand = (const char*)p.pro.operand + m0 * p.k * xbytes;
  // LDS: staged x (mt rows) + split-K partials
  const int chunk_x_bytes = cw * xbytes;
  const size_t partial_bytes = a.kw > 1 ? (size_t)a.kw * a.rows_per_wg * mt * sizeof(float) : 0;
  lds_bytes = (size_t)mt * chunk_x_bytes * a.nchunks + partial_bytes + (c.p5 == 1 ? 4 * 16 * 16 : 0);  // + the row skew
  threads = waves * 64;
  const int cus = device_cu_count();
  // resident workgroups per CU: bounded by 2048 lanes and by LDS
  int per_cu = 2048 / threads;
  const int by_lds = (int)((160 * 1024) / (lds_bytes ? lds_bytes : 1));
  if (by_lds < per_cu) per_cu = by_lds < 1 ? 1 : by_lds;
  if (per_cu < 1) per_cu = 1;
  grid = a.nblocks < cus * per_cu ? a.nblocks : cus * per_cu;
  if (grid < 1) grid = 1;
}

// One launch handles at most 4 activation rows; larger M is issued as passes of
// 4 rows (each pass streams the weights again — the MFMA variant avoids that).
int launch_gemv(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_config_applicable(p, c, &why)) return set_error(TLHIP_ERR_INVALID, "gemv: config not applicable: %s", why);
  if (p.n == 0 || p.m == 0) return TLHIP_OK;
  const int xbytes = p.x_dtype == TLHIP_F16 ? 2 : 4;

  // activation rows per pass: as many (4, 2 or 1) as fit LDS next to the partials
  int pass = 4;
  while (pass > 1 && (size_t)pass * p.k * xbytes + 16 * 1024 > (size_t)kLdsBudget) pass >>= 1;
  if (c.p5 == 1) pass = 4;  // the 4x4x4 form: four rows per pass (checked above)

  for (int64_t m0 = 0; m0 < p.m; m0 += pass) {
    const int mrows = (int)(p.m - m0 < pass ? p.m - m0 : pass);
    GemvArgs a;
    int mt, threads, grid;
    size_t lds_bytes;
    fill_args(p, c, m0, mrows, a, mt, threads, grid, lds_bytes);
    const int r = c.p1, unroll = c.p4 == 0 ? 2 : c.p4;
    int rc;
    switch (p.format) {
      case TLHIP_FMT_INT4_GROUPED:
        if (c.p5 == 1) rc = launch_gemv_mf4_int4(unroll, a, threads, grid, lds_bytes, stream);
        else rc = launch_gemv_int4(p.x_dtype, mt, r, unroll, a, threads, grid, lds_bytes, stream);
        break;
      case TLHIP_FMT_INT8_GROUPED:
        rc = launch_gemv_int8_grouped(p.x_dtype, mt, r, unroll, a, threads, grid, lds_bytes, stream);
        break;
      default:
        rc = launch_gemv_int8_row(p.x_dtype, mt, r, unroll, a, threads, grid, lds_bytes, stream);
        break;
    }
    if (rc) return rc;
    TLHIP_CHECK_HIP(hipGetLastError());
  }
  count_gemv_dispatch();
  return TLHIP_OK;
}

// Grouped launch: see gemv_grouped_kernel.  M = 1, f16 activations, and (rows per
// lane group, chunks in flight) = (1,2) or (2,2) are built.
bool gemv_group_compatible(const Problem* ps, int count, const tlhip_kernel_config_t& c, const char** why) {
  static const char* reasons[] = {
      "a group holds 1..4 problems",
      "grouped launches are built for M = 1 and f16 activations",
      "all problems of a group must share format, group size, K and output type",
      "grouped launches are built for (rows per lane group, chunks in flight) = (1,2) or (2,2)",
  };
  auto fail = [&](int i) {
    if (why) *why = reasons[i];
    return false;
  };
  if (count < 1 || count > kMaxGroup) return fail(0);
  for (int i = 0; i < count; ++i) {
    if (ps[i].m != 1 || ps[i].x_dtype != TLHIP_F16) return fail(1);
    if (ps[i].format != ps[0].format || ps[i].group_size != ps[0].group_size || ps[i].k != ps[0].k ||
        ps[i].y_dtype != ps[0].y_dtype)
      return fail(2);
    if (!gemv_config_applicable(ps[i], c, why)) return false;
  }
  const int u = c.p4 == 0 ? 2 : c.p4;
  if (u != 2 || (c.p1 != 1 && c.p1 != 2)) return fail(3);
  return true;
}

int launch_gemv_grouped(const Problem* ps, int count, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_group_compatible(ps, count, c, &why))
    return set_error(TLHIP_ERR_INVALID, "gemv_grouped: %s", why ? why : "?");
  GroupedGemvArgs g;
  g.count = 0;
  g.first[0] = 0;
  int threads = 0;
  size_t lds_bytes = 0;
  // every problem gets the workgroups it would get alone, scaled down together if
  // the sum exceeds what is resident at once
  int grids[kMaxGroup], total = 0, resident = 0;
  for (int i = 0; i < count; ++i) {
    if (ps[i].n == 0) continue;
    int mt, grid;
    size_t lds;
    fill_args(ps[i], c, 0, 1, g.p[g.count], mt, threads, grid, lds);
    lds_bytes = lds > lds_bytes ? lds : lds_bytes;
    const int cus = device_cu_count();
    int per_cu = 2048 / threads;
    const int by_lds = (int)((160 * 1024) / (lds ? lds : 1));
    if (by_lds < per_cu) per_cu = by_lds < 1 ? 1 : by_lds;
    resident = cus * per_cu;
    grids[g.count] = grid;
    total += grid;
    ++g.count;
  }
  if (g.count == 0) return TLHIP_OK;
  for (int i = 0; i < g.count; ++i) {
    int grid = grids[i];
    if (total > resident) {
      grid = (int)((int64_t)grid * resident / total);
      if (grid < 1) grid = 1;
    }
    g.first[i + 1] = g.first[i] + grid;
  }
  int rc;
  const int r = c.p1;
  switch (ps[0].format) {
    case TLHIP_FMT_INT4_GROUPED: rc = launch_gemv_grouped_int4(r, g, threads, lds_bytes, stream); break;
    case TLHIP_FMT_INT8_GROUPED: rc = launch_gemv_grouped_int8_grouped(r, g, threads, lds_bytes, stream); break;
    default: rc = launch_gemv_grouped_int8_row(r, g, threads, lds_bytes, stream); break;
  }
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  for (int i = 0; i < g.count; ++i) count_gemv_dispatch();
  return TLHIP_OK;
}

// Every instance the launch tables above can reach, in prepare mode (see launch_kernel).
int prepare_gemv_kernels() {
  GemvArgs a;
  memset(&a, 0, sizeof a);
  GroupedGemvArgs g;
  memset(&g, 0, sizeof g);
  g.count = 1;
  g.first[1] = 1;
  static const int ru[][2] = {{1, 2}, {1, 4}, {1, 8}, {2, 2}, {2, 4}, {4, 2}};
  for (int xd : {TLHIP_F16, TLHIP_F32})
    for (int mt : {1, 2, 4})
      for (auto& c : ru) {
        int rc = launch_gemv_int4(xd, mt, c[0], c[1], a, 64, 1, 0, nullptr);
        if (!rc) rc = launch_gemv_int8_grouped(xd, mt, c[0], c[1], a, 64, 1, 0, nullptr);
        if (!rc) rc = launch_gemv_int8_row(xd, mt, c[0], c[1], a, 64, 1, 0, nullptr);
        if (rc) return rc;
      }
  for (int u : {2, 4, 8}) {
    const int rc = launch_gemv_mf4_int4(u, a, 64, 1, 0, nullptr);
    if (rc) return rc;
  }
  for (int r : {1, 2}) {
    int rc = launch_gemv_grouped_int4(r, g, 64, 0, nullptr);
    if (!rc) rc = launch_gemv_grouped_int8_grouped(r, g, 64, 0, nullptr);
    if (!rc) rc = launch_gemv_grouped_int8_row(r, g, 64, 0, nullptr);
    if (rc) return rc;
  }
  return TLHIP_OK;
}

}  // namespace tlhip
