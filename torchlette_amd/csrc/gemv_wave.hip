// Host side of the per-wave pipelined skinny GEMV (gemv_wave_kernel.h): configuration
// checks, launch geometry and the kernel instances.
#include "gemv_wave_kernel.h"

namespace tlhip {
namespace {

constexpr int kWaveRpMax = 4;

struct WaveGeometry {
  int grid, rp, mq, steps, nsteps, spr, nsl, wave_units;
  size_t lds_bytes;
};

// waves per workgroup, workgroups per CU, iterations per step, whole-line weight loads ->
// geometry of one problem; false if it does not fit (more than 4 row blocks per workgroup,
// more scale pieces than the kernel loads, LDS).  The grid is the smallest that keeps the
// row blocks per workgroup, so that they divide evenly (576 row blocks: 192 workgroups of
// 3, not 256 of which 64 take 3).
bool wave_geometry(const Problem& p, int waves, int per_cu, int unroll, bool line, WaveGeometry* out, int* why) {
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  const int64_t nblocks = (p.n + 15) / 16;
  int64_t grid = (int64_t)cus * per_cu;
  if (grid > nblocks) grid = nblocks;
  if (grid < 1) grid = 1;
  const int64_t rp = (nblocks + grid - 1) / grid;
  if (rp > kWaveRpMax) return *why = 8, false;
  grid = (nblocks + rp - 1) / rp;
  const int rows_per_load = 4 / unroll;
  int mq = 1;
  while (mq * rows_per_load < p.m) mq *= 2;
  out->grid = (int)grid;
  out->rp = (int)rp;
  out->mq = mq;
  out->nsteps = (int)(p.k / (128 * unroll));
  out->steps = (out->nsteps + waves - 1) / waves;
  out->spr = (out->steps * 8 * unroll + 15) / 16;
  out->nsl = (int)((rp * 16 * out->spr + 63) / 64);
  if (out->nsl > kWaveScaleLoads || out->spr > 24) return *why = 9, false;
  out->wave_units = 16 * (16 * unroll + 1) + (line ? 128 : 0) + out->nsl * 64;
  out->lds_bytes = (size_t)waves * out->wave_units * 16 + (size_t)waves * rp * 1024;
  if (out->lds_bytes > 160 * 1024) return *why = 6, false;  // workgroups that do not fit a CU together take turns
  return true;
}

// The instances that fit the register file without spilling.
constexpr bool wave_built(int rp, int mq, int depth, int unroll, bool line) {
  const int ring = (mq * 4 + rp * unroll * 4) * depth;  // registers of the ring
  const int budget = unroll == 1 ? 92 : (!line ? 88 : (rp == 1 ? 96 : (rp == 2 ? 80 : (rp == 3 ? 64 : 56))));
  return ring <= budget && mq * (4 / unroll) <= 16;
}

template <int RP, int MQ, int D, int U, bool LINE>
const void* wave_instance() {
  if constexpr (wave_built(RP, MQ, D, U, LINE)) return (const void*)gemv_wave_kernel<RP, MQ, D, U, LINE>;
  else return nullptr;
}
template <int RP, int MQ, int U, bool LINE>
const void* wave_by_depth(int depth) {
  switch (depth) {
    case 2: return wave_instance<RP, MQ, 2, U, LINE>();
    case 3: return wave_instance<RP, MQ, 3, U, LINE>();
    case 4: return wave_instance<RP, MQ, 4, U, LINE>();
  }
  return nullptr;
}
template <int RP, int U, bool LINE>
const void* wave_by_mq(int mq, int depth) {
  switch (mq) {
    case 1: return wave_by_depth<RP, 1, U, LINE>(depth);
    case 2: return wave_by_depth<RP, 2, U, LINE>(depth);
    case 4: return wave_by_depth<RP, 4, U, LINE>(depth);
    case 8:
      if constexpr (U == 2) return wave_by_depth<RP, 8, U, LINE>(depth);
      else return nullptr;
  }
  return nullptr;
}
template <int U, bool LINE>
const void* wave_by_rp(int rp, int mq, int depth) {
  switch (rp) {
    case 1: return wave_by_mq<1, U, LINE>(mq, depth);
    case 2: return wave_by_mq<2, U, LINE>(mq, depth);
    case 3: return wave_by_mq<3, U, LINE>(mq, depth);
    case 4: return wave_by_mq<4, U, LINE>(mq, depth);
  }
  return nullptr;
}
const void* wave_fn(int rp, int mq, int depth, int unroll, bool line) {
  if (unroll == 1) return line ? nullptr : wave_by_rp<1, false>(rp, mq, depth);
  if (unroll == 2) return line ? wave_by_rp<2, true>(rp, mq, depth) : wave_by_rp<2, false>(rp, mq, depth);
  return nullptr;
}

const char* const kWaveReasons[] = {
    "not the gemv_wave variant",
    "built for int4 weights with group size 32 and f16 activations",
    "M must be 1..16",
    "waves per workgroup must be 4 or 8; steps in flight 2, 3 or 4; workgroups per CU 1 or 2; iterations per step 1 or 2; "
    "whole-line weight loads (p5 = 1) with 2 iterations per step",
    "K must be a multiple of 128 (256 with two iterations per step)",
    "weights, scales and activations must each be below 2 GiB",
    "the waves' patches and parked tiles do not fit LDS",
    "this many steps in flight need more registers than a lane has (for these rows, row blocks per workgroup and iterations per step)",
    "more than 4 row blocks of 16 rows per workgroup (N above 64 x the workgroups the chip holds)",
    "K is too long for the scales of a wave's K range to be loaded up front",
};

}  // namespace

bool gemv_wave_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  auto fail = [&](int i) {
    if (why) *why = kWaveReasons[i];
    return false;
  };
  if (c.variant != VARIANT_GEMV_WAVE) return fail(0);
  if (p.format != TLHIP_FMT_INT4_GROUPED || p.group_size != 32 || p.x_dtype != TLHIP_F16) return fail(1);
  if (p.m < 1 || p.m > 16) return fail(2);
  const int per_cu = c.p2 < 1 ? 1 : c.p2;
  const int unroll = c.p3 < 1 ? 1 : c.p3;
  if ((c.p0 != 4 && c.p0 != 8) || c.p1 < 2 || c.p1 > 4 || (per_cu != 1 && per_cu != 2) || unroll > 2 || c.p4 != 0 ||
      (c.p5 != 0 && c.p5 != 1) || (c.p5 == 1 && unroll != 2) || c.p6 != 0)
    return fail(3);
  if (p.k <= 0 || p.k % (128 * unroll) != 0) return fail(4);
  const int64_t lim = (int64_t)1 << 31;
  if (p.n * (p.k / 2) >= lim || p.m * p.k * 2 >= lim) return fail(5);
  WaveGeometry geo;
  int w = 6;
  if (!wave_geometry(p, c.p0, per_cu, unroll, c.p5 == 1, &geo, &w)) return fail(w);
  if (!wave_fn(geo.rp, geo.mq, c.p1, unroll, c.p5 == 1)) return fail(7);
  return true;
}

int launch_gemv_wave(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_wave_config_applicable(p, c, &why))
    return set_error(TLHIP_ERR_INVALID, "gemv_wave: config not applicable: %s", why);
  if (p.n == 0 || p.m == 0) return TLHIP_OK;
  const int waves = c.p0, depth = c.p1, per_cu = c.p2 < 1 ? 1 : c.p2, unroll = c.p3 < 1 ? 1 : c.p3;
  const bool line = c.p5 == 1;
  WaveGeometry geo;
  int w = 0;
  wave_geometry(p, waves, per_cu, unroll, line, &geo, &w);
  WaveArgs a;
  memset(&a, 0, sizeof a);
  a.packed = p.packed;
  a.scales = p.scales;
  a.x = p.x;
  a.y = p.y;
  a.n = (int)p.n;
  a.m = (int)p.m;
  a.kb = (int)(p.k / 2);
  a.nsteps = geo.nsteps;
  a.steps = geo.steps;
  a.spr = geo.spr;
  a.spr_recip = (65536 + geo.spr - 1) / geo.spr;
  a.nsl = geo.nsl;
  a.wave_units = geo.wave_units;
  a.packed_bytes = (uint32_t)(p.n * (p.k / 2));
  a.scales_bytes = (uint32_t)(p.n * (p.k / 32) * 2);
  a.x_bytes = (uint32_t)(p.m * p.k * 2);
  a.alpha = p.alpha;
  a.y_dtype = p.y_dtype;
  a.epi = p.epi;
  const void* fn = wave_fn(geo.rp, geo.mq, depth, unroll, line);
  if (!fn) return set_error(TLHIP_ERR_INVALID, "gemv_wave: no kernel instance for this configuration");
  void* args[] = {(void*)&a};
  const int rc = launch_kernel(fn, dim3(geo.grid), dim3(waves * 64), args, geo.lds_bytes, stream);
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  count_gemv_dispatch();
  return TLHIP_OK;
}

int prepare_gemv_wave_kernels() {
  for (int rp = 1; rp <= kWaveRpMax; ++rp)
    for (int mq : {1, 2, 4, 8})
      for (int depth = 2; depth <= 4; ++depth)
        for (int unroll = 1; unroll <= 2; ++unroll)
          for (int line = 0; line <= 1; ++line) {
            const void* fn = wave_fn(rp, mq, depth, unroll, line == 1);
            if (!fn) continue;
            const int rc = launch_kernel(fn, dim3(1), dim3(64), nullptr, 0, nullptr);
            if (rc) return rc;
          }
  return TLHIP_OK;
}

}  // namespace tlhip
