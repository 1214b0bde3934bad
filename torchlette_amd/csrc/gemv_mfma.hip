// Host side of the skinny matrix-core GEMV (gemv_mfma_kernel.h): configuration checks,
// launch geometry, the single and the grouped launch, and the single-problem kernel
// instances.  The instances with a problem table are in gemv_mfma_group.hip.
#include "gemv_mfma_kernel.h"

namespace tlhip {
static constexpr size_t kXLdsBudget = 160 * 1024;

// Grid and LDS of a launch.  With kw > 1 every workgroup parks one tile per
// (round, wave) in LDS, so LDS grows with the rounds a workgroup walks, the rounds
// shrink with the grid, and the grid is bounded by what LDS lets reside: take the
// most workgroups per CU for which it closes.
struct MfmaGeometry {
  int grid;
  size_t lds_bytes;
  size_t patch_offset;  // bytes of activations and parked tiles in front of the patches
};
// Tiles of 16 activation rows per weight row block: 1, 2 or 4 (M <= 16 / 32 / 64).
static int row_tiles(int64_t m) { return m <= 16 ? 1 : (m <= 32 ? 2 : 4); }

// `slice_k`: activations of one K slice per row (the longest slice).
static bool mfma_geometry(int64_t nblocks, int64_t slice_k, int64_t m, int waves, int kw, int ks, size_t patch_bytes, MfmaGeometry* out) {
  const int threads = waves * 64;
  const int blocks_per_wg = waves / kw;
  const int64_t nwgblocks = (nblocks + blocks_per_wg - 1) / blocks_per_wg;
  const size_t x_bytes = (size_t)m * (slice_k * 2 + 16);
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  for (int per_cu = 2048 / threads; per_cu >= 1; --per_cu) {
    int64_t sets = (int64_t)cus * per_cu / ks;
    // A wave that owns its row blocks (no K split): twice the workgroups the chip holds
    // at a time, each walking half as many blocks.  The second half starts as the first
    // finishes, which evens out the workgroups' different speeds: 2-3 % on the LM head
    // (256 000 rows, M = 3..16), although every workgroup stages the activations anew.
    if (kw == 1 && ks == 1) sets *= 2;
    if (sets > nwgblocks) sets = nwgblocks;
    if (sets < 1) sets = 1;
    const int64_t rounds = (nwgblocks + sets - 1) / sets;
    const size_t parked = kw > 1 ? (size_t)rounds * waves * 1024 * row_tiles(m) : 0;
    const size_t lds = x_bytes + parked + patch_bytes;
    if (lds * per_cu <= kXLdsBudget) {
      out->grid = (int)(sets * ks);
      out->lds_bytes = lds;
      out->patch_offset = x_bytes + parked;
      return true;
    }
  }
  return false;
}

// LDS of the wave-private patches of the whole-line form: 2 KB per pair of iterations.
static size_t line_patch_bytes(const tlhip_kernel_config_t& c) {
  return c.p5 == 1 ? (size_t)c.p0 * c.p1 * 1024 : 0;
}

// `nblocks`: 16-row blocks of the launch (of all problems of a group together).
static bool mfma_applicable(const Problem& p, int64_t nblocks, const tlhip_kernel_config_t& c, const char** why) {
  static const char* reasons[] = {
      "not the gemv_mfma variant",
      "waves per workgroup must be 4, 8 or 16 (16: at most two iterations in flight)",
      "activations must be f16",
      "M must be 1..16 (17..64 for one problem with at most 8 waves per workgroup)",
      "K must be a multiple of 128 (int4) or 64 (int8)",
      "group size must be a multiple of 32 (int4) or 64 (int8)",
      "iterations in flight must be 1, 2 or 4 (1 or 2 above 32 rows)",
      "K-split waves must be a power of two that divides the waves per workgroup",
      "activations (M x K/slices f16) plus one parked tile per round and wave do not fit LDS",
      "K slices must be a power of two (1..16) that divides K/128 (int4) or K/64 (int8); slices of unequal length "
      "(any power of two up to the step count) take one iteration in flight and no whole-line loads",
      "K slices need more partial-tile workspace or counters than the library holds",
      "iterations in flight must divide the 128-weight (int4) or 64-weight (int8) steps of a K slice",
      "whole-line weight loads (p5 = 1) need int8 (K % 128 == 0) or int4 with group size 32 "
      "(K % 256 == 0), 2 or 4 iterations in flight and an even number of iterations per K slice",
  };
  auto fail = [&](int i) {
    if (why) *why = reasons[i];
    return false;
  };
  if (c.variant != VARIANT_GEMV_MFMA) return fail(0);
  if (c.p0 != 4 && c.p0 != 8 && c.p0 != 16) return fail(1);
  if (c.p0 == 16 && c.p1 > 2) return fail(1);
  if (p.x_dtype != TLHIP_F16) return fail(2);
  if (p.m < 1 || p.m > 64) return fail(3);
  if (p.m > 16 && c.p0 > 8) return fail(3);
  if (p.m > 32 && c.p1 > 2) return fail(6);  // four tiles of rows and four iterations in flight: more registers than a lane has
  const int kper = p.format == TLHIP_FMT_INT4_GROUPED ? 128 : 64;
  if (p.k % kper != 0) return fail(4);
  if (p.format == TLHIP_FMT_INT4_GROUPED && p.group_size % 32 != 0) return fail(5);
  if (p.format == TLHIP_FMT_INT8_GROUPED && p.group_size % 64 != 0) return fail(5);
  if (c.p1 != 1 && c.p1 != 2 && c.p1 != 4) return fail(6);
  const int kw = c.p2 == 0 ? c.p0 : c.p2;
  if (kw < 1 || (kw & (kw - 1)) != 0 || c.p0 % kw != 0) return fail(7);
  const int ks = c.p3 < 1 ? 1 : c.p3;
  const int64_t iters = p.k / kper;
  if (ks > 16 || (ks & (ks - 1)) != 0 || ks > iters) return fail(9);
  const bool uneven = iters % ks != 0;
  if (uneven && (c.p1 != 1 || c.p5 != 0)) return fail(9);
  const int64_t slice_k = (iters / ks + (uneven ? 1 : 0)) * kper;  // the longest slice
  if (c.p5 != 0) {
    // a pair of iterations = one 128-byte line per row: 128 k of int8, 256 k of int4
    const bool fmt_ok = ((p.format == TLHIP_FMT_INT8_ROW || p.format == TLHIP_FMT_INT8_GROUPED) && p.k % 128 == 0) ||
                        (p.format == TLHIP_FMT_INT4_GROUPED && p.group_size == 32 && p.k % 256 == 0);
    if (!(c.p5 == 1 && fmt_ok && (c.p1 == 2 || c.p1 == 4) && !uneven && (iters / ks) % 2 == 0)) return fail(12);
  }
  MfmaGeometry geo;
  if (!mfma_geometry(nblocks, slice_k, p.m, c.p0, kw, ks, line_patch_bytes(c), &geo)) return fail(8);
  if (!uneven && (iters / ks) % c.p1 != 0) return fail(11);
  if (ks > 1 && (nblocks > scratch_counters(p) || (size_t)nblocks * ks * 256 * row_tiles(p.m) > scratch_tile_floats(p)))
    return fail(10);
  return true;
}

bool gemv_mfma_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  return mfma_applicable(p, (p.n + 15) / 16, c, why);
}

// The problems of a group: same activations and rows, one shape class; N, pointers and
// epilogues per problem.  The configuration is checked against the group's total rows.
bool gemv_mfma_group_applicable(const Problem* ps, int count, const tlhip_kernel_config_t& c, const char** why) {
  if (count < 1 || count > kMfmaMaxGroup) {
    if (why) *why = "a group holds 1..4 problems";
    return false;
  }
  int64_t nblocks = 0;
  for (int i = 0; i < count; ++i) {
    if ((count > 1 && ps[i].m > 16) || ps[i].x != ps[0].x || ps[i].m != ps[0].m || ps[i].format != ps[0].format || ps[i].group_size != ps[0].group_size ||
        ps[i].k != ps[0].k || ps[i].x_dtype != ps[0].x_dtype || ps[i].y_dtype != ps[0].y_dtype || ps[i].alpha != ps[0].alpha) {
      if (why) *why = "the problems of a group share activations, rows, format, group size, K, output type and alpha";
      return false;
    }
    nblocks += (ps[i].n + 15) / 16;
  }
  return mfma_applicable(ps[0], nblocks > 0 ? nblocks : 1, c, why);
}

int launch_gemv_mfma_group(const Problem* ps, int count, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_mfma_group_applicable(ps, count, c, &why))
    return set_error(TLHIP_ERR_INVALID, "gemv_mfma: config not applicable: %s", why);
  const Problem& p = ps[0];
  const bool int4 = p.format == TLHIP_FMT_INT4_GROUPED;
  const int cw = int4 ? 32 : 16;
  const int waves = c.p0, unroll = c.p1;
  MfmaArgs a;
  memset(&a, 0, sizeof a);
  int64_t nblocks = 0;
  for (int i = 0; i < count; ++i) {
    if (ps[i].n == 0) continue;
    MfmaProblem& P = a.p[a.count++];
    P.packed = (const u32x4*)ps[i].packed;
    P.scales = ps[i].scales;
    P.y = ps[i].y;
    P.n = ps[i].n;
    P.first_block = (int)nblocks;
    P.epi = ps[i].epi;
    nblocks += (ps[i].n + 15) / 16;
  }
  if (a.count == 0 || p.m == 0) return TLHIP_OK;
  a.x = (const _Float16*)p.x;
  a.k = (int)p.k;
  a.m = (int)p.m;
  a.nchunks = (int)(p.k / cw);
  a.cpg_shift = p.format == TLHIP_FMT_INT8_ROW ? 0 : __builtin_ctz((unsigned)(p.group_size / cw));
  a.groups_per_row = p.format == TLHIP_FMT_INT8_ROW ? 0 : (int)(p.k / p.group_size);
  a.iters = a.nchunks / 4;
  a.ks = c.p3 < 1 ? 1 : c.p3;
  a.ks_shift = __builtin_ctz((unsigned)a.ks);
  a.slice_iters = a.iters / a.ks;
  a.slice_rem = a.iters % a.ks;
  a.kw = c.p2 == 0 ? waves : c.p2;
  a.kw_shift = __builtin_ctz((unsigned)a.kw);
  a.blocks_per_wg = waves / a.kw;
  const int nbatches = a.slice_iters / unroll;
  a.nsteps = (nbatches + a.kw - 1) / a.kw;
  a.workspace = nullptr;
  a.counters = nullptr;
  if (a.ks > 1) {
    const int rc = problem_scratch(p, stream, &a.workspace, &a.counters);
    if (rc) return rc;
  }
  a.nblocks = (int)nblocks;
  a.nwgblocks = (a.nblocks + a.blocks_per_wg - 1) / a.blocks_per_wg;
  a.alpha = p.alpha;
  a.scale_mul = p.format == TLHIP_FMT_INT8_GROUPED ? (1.0f / 127.0f) : 1.0f;
  a.y_dtype = p.y_dtype;
  MfmaGeometry geo;
  const int kper = int4 ? 128 : 64;
  if (!mfma_geometry(nblocks, (int64_t)(a.slice_iters + (a.slice_rem ? 1 : 0)) * kper, p.m, waves, a.kw, a.ks, line_patch_bytes(c), &geo))
    return set_error(TLHIP_ERR_INVALID, "gemv_mfma: launch geometry does not close");
  const size_t lds_bytes = geo.lds_bytes;
  a.patch_unit = (int)(geo.patch_offset / 16);
  const int threads = waves * 64;
  const int grid = geo.grid;
  // the single-problem instances keep the problem's fields in scalar registers without a
  // table lookup per batch (measured 0.7-1.4 us per launch at the 9-28 MB decode shapes)
  int rc;
  if (p.m > 16) rc = launch_mfma_rows(row_tiles(p.m), p.format, p.group_size, p.k, unroll, c.p5, a, grid, threads, lds_bytes, stream);
  else if (a.count == 1) rc = launch_mfma_single(p.format, p.group_size, p.k, unroll, c.p5, a, grid, threads, lds_bytes, stream);
  else rc = launch_mfma_grouped(p.format, p.group_size, p.k, unroll, c.p5, a, grid, threads, lds_bytes, stream);
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  for (int i = 0; i < a.count; ++i) count_gemv_dispatch();
  return TLHIP_OK;
}

int launch_gemv_mfma(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_mfma_config_applicable(p, c, &why))
    return set_error(TLHIP_ERR_INVALID, "gemv_mfma: config not applicable: %s", why);
  if (p.n == 0 || p.m == 0) return TLHIP_OK;
  return launch_gemv_mfma_group(&p, 1, c, stream);
}

int launch_mfma_single(int format, int group_size, int64_t k, int unroll, int line, const MfmaArgs& a, int grid, int threads,
                       size_t lds_bytes, hipStream_t stream) {
  return launch_mfma_instance<false>(format, group_size, k, unroll, line, a, grid, threads, lds_bytes, stream);
}
int prepare_mfma_single() { return prepare_mfma_instances<false>(); }

int prepare_gemv_mfma_kernels() {
  int rc = prepare_mfma_single();
  if (!rc) rc = prepare_mfma_grouped();
  return rc ? rc : prepare_mfma_rows();
}

}  // namespace tlhip
