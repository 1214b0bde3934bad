// The matmul seam for packed weights and the kernel-choice machinery around it.
//
// Mirrors, for this path only:
//  * matmulQuantizedB's routing (src/backend/webgpu/ops/matmul-ops.ts:113-182):
//    the operand format is read here and nowhere above;
//  * the variant registry / selection order of
//    src/backend/webgpu/matmul/dispatch.ts:171-192: explicit config, then the
//    per-shape tuned winner (re-gated on applicability), then the first
//    applicable variant's heuristic default;
//  * the autotuner of dispatch.ts:405-547 (warm-up, then timed runs per
//    candidate, median) with a per-exact-shape cache that, unlike the
//    reference's m_n_k_dtype key, also carries the operand format, because the
//    winner differs per packing; a candidate is timed as a batch of back-to-back
//    launches per event pair (the kernels take 3-12 us: one launch per event pair
//    measures the events), with the weight rotating through alias buffers larger
//    than the last-level cache, and the three fastest are timed once more, longer;
//  * the per-shape-class level of autotune.ts:269-300: an untuned problem takes
//    the winner of the nearest tuned problem of its class before the hand
//    heuristic, and a quick tuning pass searches the neighbours of that choice
//    (generateNeighborConfigs, autotune.ts:419-465);
//  * exportTuningCache / importTuningCache (autotune.ts:309-329) as JSON text.
#include <algorithm>
#include <array>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <vector>

#include <dlfcn.h>

#include "common.h"

namespace tlhip {
namespace {

std::mutex g_tune_mutex;      // guards every variable of this block
std::mutex g_tune_run_mutex;  // held for a whole tuning run: one tuner at a time
std::map<std::string, tlhip_kernel_config_t> g_tuned;  // per exact problem key
// The shape-class level (autotune.ts:269-300): every per-shape winner is also filed under
// its class, with the shape it was found for.
struct ClassEntry {
  int64_t m, n, k;
  tlhip_kernel_config_t config;
};
std::map<std::string, std::vector<ClassEntry>> g_class_tuned;
std::vector<std::array<int64_t, 3>> g_shape_hints;
int g_autotune_counter = 0;
bool g_autotuning = false;  // no recursive tuning (dispatch.ts autotuningInProgress)

bool is_pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }

const char* format_name(int f) {
  switch (f) {
    case TLHIP_FMT_INT8_GROUPED: return "int8-grouped";
    case TLHIP_FMT_INT8_ROW: return "int8-row";
    case TLHIP_FMT_INT4_GROUPED: return "int4-grouped";
  }
  return "?";
}

std::string problem_key(const Problem& p) {
  char buf[160];
  snprintf(buf, sizeof buf, "%lld_%lld_%lld_%s_g%d_%s_%s", (long long)p.m, (long long)p.n, (long long)p.k,
           format_name(p.format), p.format == TLHIP_FMT_INT8_ROW ? 0 : p.group_size,
           p.x_dtype == TLHIP_F16 ? "f16" : "f32", p.y_dtype == TLHIP_F16 ? "f16" : "f32");
  return buf;
}

// Shape class of a problem: which kernel family serves it (rows M), what bounds it
// (bytes of packed weights: launch-, stream- or capacity-bound) and whether the
// activation rows fit one workgroup's LDS (K), per operand format and types.  The role
// of classifyShape (src/backend/webgpu/matmul/types.ts:146-200) for this path.
std::string class_key(const Problem& p) {
  const char* mc = p.m == 1 ? "m1" : p.m == 2 ? "m2" : p.m <= 4 ? "m4" : p.m <= 16 ? "m16" : p.m < 1024 ? "mid" : "big";
  const double bytes = (double)p.n * (double)p.k * (p.format == TLHIP_FMT_INT4_GROUPED ? 0.5 : 1.0);
  const char* sc = bytes < 4e6 ? "small" : bytes < 96e6 ? "medium" : "large";
  const char* kc = p.k <= 4096 ? "k4k" : p.k <= 8192 ? "k8k" : "klong";
  char buf[160];
  snprintf(buf, sizeof buf, "%s_%s_%s_%s_g%d_%s_%s", mc, sc, kc, format_name(p.format),
           p.format == TLHIP_FMT_INT8_ROW ? 0 : p.group_size, p.x_dtype == TLHIP_F16 ? "f16" : "f32",
           p.y_dtype == TLHIP_F16 ? "f16" : "f32");
  return buf;
}

// Key text -> the shape-determining fields of a Problem (what export writes).
bool parse_problem_key(const std::string& key, Problem* p) {
  long long m = 0, n = 0, k = 0;
  char fmt[32] = "", xd[8] = "", yd[8] = "";
  int g = 0;
  if (sscanf(key.c_str(), "%lld_%lld_%lld_%31[^_]_g%d_%7[^_]_%7s", &m, &n, &k, fmt, &g, xd, yd) != 7) return false;
  memset(p, 0, sizeof *p);
  if (!strcmp(fmt, "int8-grouped")) p->format = TLHIP_FMT_INT8_GROUPED;
  else if (!strcmp(fmt, "int8-row")) p->format = TLHIP_FMT_INT8_ROW;
  else if (!strcmp(fmt, "int4-grouped")) p->format = TLHIP_FMT_INT4_GROUPED;
  else return false;
  p->m = m;
  p->n = n;
  p->k = k;
  p->group_size = g;
  p->x_dtype = !strcmp(xd, "f16") ? TLHIP_F16 : TLHIP_F32;
  p->y_dtype = !strcmp(yd, "f16") ? TLHIP_F16 : TLHIP_F32;
  p->alpha = 1.f;
  return true;
}

// Caller holds g_tune_mutex.
void record_winner_locked(const Problem& p, const tlhip_kernel_config_t& c) {
  g_tuned[problem_key(p)] = c;
  auto& list = g_class_tuned[class_key(p)];
  for (auto& e : list)
    if (e.m == p.m && e.n == p.n && e.k == p.k) {
      e.config = c;
      return;
    }
  list.push_back({p.m, p.n, p.k, c});
}

bool env_autotune() {
  const char* e = getenv("TORCHLETTE_AUTOTUNE");
  return e && !strcmp(e, "1");
}

tlhip_kernel_config_t gemv_cfg(int lpr, int r, int waves, int kw, int unroll) {
  tlhip_kernel_config_t c;
  memset(&c, 0, sizeof c);
  c.variant = VARIANT_GEMV;
  c.p0 = lpr;
  c.p1 = r;
  c.p2 = waves;
  c.p3 = kw;
  c.p4 = unroll;
  return c;
}

tlhip_kernel_config_t mfma_cfg(int waves, int unroll, int kw, int ks = 1) {
  tlhip_kernel_config_t c;
  memset(&c, 0, sizeof c);
  c.variant = VARIANT_GEMV_MFMA;
  c.p0 = waves;
  c.p1 = unroll;
  c.p2 = kw;
  c.p3 = ks;
  return c;
}

tlhip_kernel_config_t xreg_cfg(int waves, int unroll, int per_cu, int ks, int upfront = 0, int xbar = 0) {
  tlhip_kernel_config_t c;
  memset(&c, 0, sizeof c);
  c.variant = VARIANT_GEMV_XREG;
  c.p0 = waves;
  c.p1 = unroll;
  c.p2 = per_cu;
  c.p3 = ks;
  c.p4 = upfront;
  c.p5 = xbar;
  return c;
}

tlhip_kernel_config_t wave_cfg(int waves, int depth, int per_cu, int unroll) {
  tlhip_kernel_config_t c;
  memset(&c, 0, sizeof c);
  c.variant = VARIANT_GEMV_WAVE;
  c.p0 = waves;
  c.p1 = depth;
  c.p2 = per_cu;
  c.p3 = unroll;
  return c;
}

tlhip_kernel_config_t tiled_cfg(int tm, int tn, int tk, int wm, int wn) {
  tlhip_kernel_config_t c;
  memset(&c, 0, sizeof c);
  c.variant = VARIANT_TILED;
  c.p0 = tm;
  c.p1 = tn;
  c.p2 = tk;
  c.p3 = wm;
  c.p4 = wn;
  return c;
}

tlhip_kernel_config_t direct_cfg(int tm, int tn, int wm, int wn) {
  tlhip_kernel_config_t c = tiled_cfg(tm, tn, 128, wm, wn);
  c.variant = VARIANT_TILED_DIRECT;
  return c;
}


bool config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  if (c.variant == VARIANT_TILED_DIRECT) return gemm_direct_config_applicable(p, c, why);
  if (c.variant == VARIANT_TILED) return gemm_config_applicable(p, c, why);
  if (c.variant == VARIANT_GEMV_MFMA) return gemv_mfma_config_applicable(p, c, why);
  if (c.variant == VARIANT_GEMV_XREG) return gemv_xreg_config_applicable(p, c, why);
  if (c.variant == VARIANT_GEMV_WAVE) return gemv_wave_config_applicable(p, c, why);
  return gemv_config_applicable(p, c, why);
}

tlhip_kernel_config_t default_valu_config(const Problem& p);

// The numbers the default routing was fitted with on MI355X: measurements, not structure.
// They live next to the tuned entries: the tuning file may carry a "model" object that
// overrides any of them by name (tlhip_tune_cache_import), the export writes them back,
// and tlhip_tune_cache_clear returns to the built-in values below.
struct RouteModel {
  double walk_direct_us = 42.0;      // a workgroup of the direct GEMM walks 4096 of K in this time
  double walk_staged128_us = 52.0;   // ... of the staged GEMM's 128-row tile
  double walk_staged64_us = 42.0;    // ... of its 64-row tile
  double reduce_base_us = 6.0;       // the launch that adds K slices: base
  double reduce_us_per_mb = 0.6;     // ... per MB of f32 planes
  double crowd_base = 0.45;          // rounds of a crowded launch: base + slope x (workgroups / CUs)
  double crowd_slope = 0.78;
  double pass_base_us = 3.0;         // a 16-row pass of the decode kernel: base
  double pass_mb_per_us = 3.2;       // ... plus packed MB / this
  double rows32_factor = 1.5;        // 17..32 rows in one launch of the decode kernel, in 16-row passes
  double rows64_factor = 2.7;        // 33..64 rows
  double rows_break_even = 0.9;      // rows through the decode kernel while below this x the tiled time
  double passes_break_even = 0.8;    // 16-row passes while below this x the tiled time
  double resident_tiles = 512.0;     // 128 x 128 tiles that run at once
  double int4_256_rounds = 2.0;      // int4: 256 x 256 tiles from this many per CU on
  double int4_128x256_tiles = 160.0; // int4: 128 x 256 tiles from this many on
  double int8_256_fill = 0.5625;     // int8: 256 x 256 tiles once they are this fraction of the CUs
  double int8_256x128_fill = 0.625;  // int8: 256 x 128 tiles likewise
  double int8_row_fill = 0.58;       // int8 direct kernel only if the rows fill this much of their 256-row tiles
  double binary_tail_elements = 4000000.0;  // a binary step on M x N outputs from this size on runs behind the GEMM
};
RouteModel g_model;
struct ModelField {
  const char* name;
  double RouteModel::*field;
};
const ModelField kModelFields[] = {
    {"walk_direct_us", &RouteModel::walk_direct_us},       {"walk_staged128_us", &RouteModel::walk_staged128_us},
    {"walk_staged64_us", &RouteModel::walk_staged64_us},   {"reduce_base_us", &RouteModel::reduce_base_us},
    {"reduce_us_per_mb", &RouteModel::reduce_us_per_mb},   {"crowd_base", &RouteModel::crowd_base},
    {"crowd_slope", &RouteModel::crowd_slope},             {"pass_base_us", &RouteModel::pass_base_us},
    {"pass_mb_per_us", &RouteModel::pass_mb_per_us},       {"rows32_factor", &RouteModel::rows32_factor},
    {"rows64_factor", &RouteModel::rows64_factor},         {"rows_break_even", &RouteModel::rows_break_even},
    {"passes_break_even", &RouteModel::passes_break_even}, {"resident_tiles", &RouteModel::resident_tiles},
    {"int4_256_rounds", &RouteModel::int4_256_rounds},     {"int4_128x256_tiles", &RouteModel::int4_128x256_tiles},
    {"int8_256_fill", &RouteModel::int8_256_fill},         {"int8_256x128_fill", &RouteModel::int8_256x128_fill},
    {"int8_row_fill", &RouteModel::int8_row_fill},
    {"binary_tail_elements", &RouteModel::binary_tail_elements},
};

// Time of one round of 128 x 128 tiles of the direct GEMM with `ks` K slices across
// workgroups, in microseconds: a workgroup walks 4096 of K in 42 us; the slices' partial
// sums (ks planes of M x N f32) are written and read back by a second launch, 6 us plus
// 0.6 us per MB of planes (fitted at 4096..12288 x 4096..12288, M = 64..512).
double direct_round_us(const Problem& p, int ks, double walk_4096_us) {
  const double walk = walk_4096_us * (double)p.k / 4096.0 / ks;
  if (ks <= 1) return walk;
  return walk + g_model.reduce_base_us + g_model.reduce_us_per_mb * (double)ks * (double)p.m * (double)p.n * 4.0 / 1e6;
}

// Time of a launch of the staged GEMM's 128 x 128 or 64 x 128 tiles by the same model, in
// microseconds: a round of the 128-row tiles walks 4096 of K in 52 us, of the 64-row tiles
// in 42 us; x = tiles x slices / CUs up to 1 is one round, beyond that 0.45 + 0.78 x rounds
// (workgroups that share a CU slow each other down: measured 1.38 / 1.56 / 1.83 / 2.73 / 5.2
// rounds at x = 1.125 / 1.5 / 2 / 3 / 6).
double staged_launch_us(const Problem& p, const tlhip_kernel_config_t& c) {
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  const int ks = c.p5 > 1 ? c.p5 : 1;
  const int64_t tiles = ((p.m + c.p0 - 1) / c.p0) * ((p.n + c.p1 - 1) / c.p1);
  const double fill = (double)(tiles * ks) / (double)cus;
  const double rounds = fill <= 1.0 ? 1.0 : g_model.crowd_base + g_model.crowd_slope * fill;
  const double walk_us = (c.p0 <= 64 ? g_model.walk_staged64_us : g_model.walk_staged128_us) * (double)p.k / 4096.0 / ks;
  const double sum_us = direct_round_us(p, ks, 0.0);  // the second launch of a K-sliced one
  return rounds * walk_us + sum_us;
}

// K slices across workgroups for a launch of 128 x 128 tiles of the direct GEMM: of 1, 2,
// 4, 8 the cheapest by direct_round_us that keeps tiles x slices within the CUs (beyond,
// the slices of a tile queue behind each other), divides the 128-k steps and leaves every
// slice at least four of them.
int direct_k_split(const Problem& p) {
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  const int64_t tiles = ((p.m + 127) / 128) * ((p.n + 127) / 128);
  const int64_t steps = p.k / 128;
  int best = 1;
  for (int ks = 2; ks <= 8; ks *= 2)
    if (tiles * ks <= cus && steps % ks == 0 && steps / ks >= 4 && direct_round_us(p, ks, g_model.walk_direct_us) < direct_round_us(p, best, g_model.walk_direct_us)) best = ks;
  return best;
}

// Heuristic default, used when nothing is tuned.
tlhip_kernel_config_t default_config(const Problem& p) {
  if (p.m > 16 && p.x_dtype == TLHIP_F16) {
    const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
    // int4: the kernel that keeps the weights packed up to the operand registers.
    // Tiles by how many there are (best of every tile at 2048..28672 x 2048..12288, M =
    // 32..4096): 256 x 256 once they fill the chip twice over; 128 x 256 with four waves
    // (two workgroups share a CU) from 160 such tiles on, never more than 7 % behind the
    // best there; below that 128 x 128, where the 256-row tiles measured 1.4-1.5 times
    // slower (a launch of few tiles takes the time one workgroup needs to walk K).
    if (p.format == TLHIP_FMT_INT4_GROUPED) {
      const int64_t t256 = ((p.m + 255) / 256) * ((p.n + 255) / 256);
      const int64_t t128x256 = ((p.m + 127) / 128) * ((p.n + 255) / 256);
      tlhip_kernel_config_t c = (double)t256 >= g_model.int4_256_rounds * cus
                                    ? direct_cfg(256, 256, 2, 4)
                                    : ((double)t128x256 >= g_model.int4_128x256_tiles ? direct_cfg(128, 256, 1, 4) : direct_cfg(128, 128, 2, 2));
      if (c.p0 == 128 && c.p1 == 128) {
        // few 128 x 128 tiles: 2, 4 or 8 workgroups share a tile, each walking a slice of K
        // of at least four steps (4096 x 12288 at M = 256: 48 us against 141 us)
        const int ks = direct_k_split(p);
        if (ks > 1) {
          tlhip_kernel_config_t split = c;
          split.p5 = ks;
          if (gemm_direct_config_applicable(p, split, nullptr)) return split;
        }
      }
      if (gemm_direct_config_applicable(p, c, nullptr)) return c;
    }
    // int8 per row, or in groups of 64 or more: the same kernel once its 256-row tiles fill
    // the chip (2048..28672 x 2048..14336, M = 32..8192, per row and groups of 64 and 128:
    // the 256 x 256 tile was the best of every tile of both kernels from 144 tiles on, 4-27 %
    // ahead of the staged kernel; 256 x 128 from 160 tiles on, 3-15 % ahead); with fewer
    // tiles the staged kernel below is ahead by 3-40 %.  Not where the rows fill less than
    // 58 % of their 256-row tiles (128 rows on 28672 columns: 78 us against 52 us).
    if ((p.format == TLHIP_FMT_INT8_GROUPED || p.format == TLHIP_FMT_INT8_ROW) &&
        (double)p.m >= (double)(((p.m + 255) / 256) * 256) * g_model.int8_row_fill) {
      const int64_t t256 = ((p.m + 255) / 256) * ((p.n + 255) / 256);
      const int64_t t256x128 = ((p.m + 255) / 256) * ((p.n + 127) / 128);
      if ((double)t256 >= g_model.int8_256_fill * cus) {
        const tlhip_kernel_config_t c = direct_cfg(256, 256, 2, 4);
        if (gemm_direct_config_applicable(p, c, nullptr)) return c;
      } else if ((double)t256x128 >= g_model.int8_256x128_fill * cus) {
        const tlhip_kernel_config_t c = direct_cfg(256, 128, 2, 4);
        if (gemm_direct_config_applicable(p, c, nullptr)) return c;
      }
    }
    // The LDS-staged kernel (the int8 formats): the 128 x 128 or the 64 x 128 tile, with K
    // slices across workgroups where the tiles are few, whichever the model of a launch
    // prices lowest: tiles x slices / CUs rounds (at least one) of the time a workgroup
    // needs to walk its slice (52 us per 4096 of K for the 128-row tile, 42 us for the
    // 64-row tile) plus the second launch that adds the slices.  Within 10 % of the best
    // of every tile and slice count at 2048..28672 x 2048..14336, M = 32..2048; the 256 x
    // 128 tile was up to 42 % slower.
    {
      tlhip_kernel_config_t best_c{};
      double best_us = 0.0;
      bool have = false;
      for (const int bm : {128, 64}) {
        const int64_t wgs = ((p.m + bm - 1) / bm) * ((p.n + 127) / 128);
        const tlhip_kernel_config_t c = tiled_cfg(bm, 128, 64, 2, 2);
        if (!gemm_config_applicable(p, c, nullptr)) continue;
        for (int ks = 1; ks <= 8; ks *= 2) {
          tlhip_kernel_config_t split = c;
          if (ks > 1) {
            // every slice at least 512 of K, and at most two workgroups to a CU (the model
            // prices the crowding: 160 rows at 5120 x 5120 took 36 us in 4 slices, 320
            // workgroups, against 42 us in 2)
            if (wgs * ks > 2 * cus || (p.k / 64) % ks != 0 || p.k / ks < 512) continue;
            split.p5 = ks;
            if (!gemm_config_applicable(p, split, nullptr)) continue;
          }
          const double us = staged_launch_us(p, split);
          if (!have || us < best_us) {
            best_c = split;
            best_us = us;
            have = true;
          }
        }
      }
      if (have) return best_c;
    }
  }
  // three or four rows of int4 weights with K up to 8192, from 8 MB of weights on: the
  // VALU kernel's 4x4x4 matrix-core form (tuned winner at 5120..14336 x 4096..8192:
  // 7.8-12.2 us against 9.9-15.7 us for the skinny kernel below, which is ahead for
  // longer K and for smaller matrices: 3584 x 3584 took 5.2 against 6.7 us)
  const double packed_mb = (double)p.n * (double)p.k * (p.format == TLHIP_FMT_INT4_GROUPED ? 0.5 : 1.0) / 1e6;
  if (p.m >= 3 && p.m <= 4 && p.k <= 8192 && packed_mb >= 8.0) {
    for (int waves : {8, 4}) {
      tlhip_kernel_config_t c = gemv_cfg(16, 1, waves, 1, 2);
      c.p5 = 1;
      if (gemv_config_applicable(p, c, nullptr)) return c;
    }
  }
  // three or more activation rows: the matrix-core kernel, whose time hardly depends on
  // M (measured at the Qwen3-8B shapes: M = 4 takes 5.3 / 10.9 / 11.2 us against 7.5 /
  // 13.4 / 15.1 us for the VALU kernel, whose dot products grow with M; at M = 2 the VALU
  // kernel is still ahead, 5.3 / 8.9 / 9.9 against 6.0 / 10.3 / 11.5 us)
  if (p.m >= 3 && p.m <= 16) {
    // a long int8 matrix (an LM head): the form with whole-line weight loads
    if ((p.format == TLHIP_FMT_INT8_ROW || p.format == TLHIP_FMT_INT8_GROUPED) && p.n >= 32768)
      for (int unroll : {4, 2}) {
        tlhip_kernel_config_t c = mfma_cfg(8, unroll, 1, 1);
        c.p5 = 1;
        if (gemv_mfma_config_applicable(p, c, nullptr)) return c;
      }
    // the fewest K slices across workgroups whose activations fit LDS (measured best);
    // the preferred split of K over a workgroup's waves first, then whatever closes (the
    // tiles the waves park in LDS grow with the rounds a workgroup walks: K = 18944 at
    // M = 16 fits with two K-split waves and not with four)
    // int8 weights (a byte per weight: 16..50 MB at the Qwen3-8B shapes) stream faster with
    // whole-line loads, four iterations in flight where they fit (tuned winner for all
    // three int8 formats at M = 4..16: 12.0-14.6 us against 14.2-17.4 us without)
    const bool int8 = p.format != TLHIP_FMT_INT4_GROUPED;
    // first the full form (eight or four K-split waves, four iterations in flight) with as
    // few K slices as let it fit: where 16 rows of K = 4096 leave no room for it in one
    // slice, two slices take 14.4-14.7 us at 12288 x 4096 against 16.8-17.7 us for what
    // does fit in one (two K-split waves, two iterations in flight)
    if (int8 && p.n < 32768)
      for (int ks = 1; ks <= 4; ks *= 2)
        for (int i = 0; i < 2; ++i) {
          // eight K-split waves first, four first where a workgroup walks a slice of more than 2048 of K
          const int kw = (ks > 1 && p.k / ks > 2048) == (i == 0) ? 4 : 8;
          tlhip_kernel_config_t c = mfma_cfg(8, 4, kw, ks);
          c.p5 = 1;
          if (gemv_mfma_config_applicable(p, c, nullptr)) return c;
        }
    if (int8)
      for (int ks = 1; ks <= 4; ks *= 2) {  // one more K slice rather than no whole-line loads (14.3 against 17.4 us)
        const int preferred = p.n >= 32768 ? 1 : (ks > 1 ? 4 : 8);
        for (int kw : {preferred, 8, 4, 2, 1})
          for (int unroll : {4, 2}) {
            tlhip_kernel_config_t c = mfma_cfg(8, unroll, kw, ks);
            c.p5 = 1;
            if (gemv_mfma_config_applicable(p, c, nullptr)) return c;
          }
      }
    for (int ks = 1; ks <= 16; ks *= 2) {
      const int preferred = p.n >= 32768 ? 1 : (ks > 1 ? 4 : 8);
      for (int kw : {preferred, 8, 4, 2, 1}) {
        for (int unroll : {2, 1, 4}) {
          tlhip_kernel_config_t c = mfma_cfg(8, unroll, kw, ks);
          if (gemv_mfma_config_applicable(p, c, nullptr)) return c;
        }
      }
    }
    // no geometry of the LDS-staged kernel closes: the activations in registers
    for (int ks = 1; ks <= 16; ks *= 2)
      for (int waves : {8, 4, 16}) {
        tlhip_kernel_config_t c = xreg_cfg(waves, 1, 1, ks);
        if (gemv_xreg_config_applicable(p, c, nullptr)) return c;
      }
  }
  return default_valu_config(p);
}

// Heuristic default of the VALU kernel (the only one for M <= 4, and the one the
// prologue entry points use).
tlhip_kernel_config_t default_valu_config(const Problem& p) {
  const int cw = p.format == TLHIP_FMT_INT4_GROUPED ? 32 : 16;
  const int64_t nchunks = p.k / cw;
  if (p.n >= 32768) {
    // long weight matrices (an LM head): 16 lanes per row, more rows per wave, walked
    // with a stride, all chunks of a row in flight at once
    const int per_lane = (int)((nchunks + 15) / 16);
    const int unroll = per_lane >= 8 ? 8 : (per_lane >= 4 ? 4 : 2);
    const int r = unroll <= 2 ? 4 : (unroll <= 4 ? 2 : 1);
    return gemv_cfg(16, r, 8, 1, unroll);
  }
  // Lanes per row and chunks in flight, from the tuned winners at 2048..18944 x
  // 2048..18944 (M = 1): 16 lanes per row up to K = 4096 and 32 beyond, two chunks
  // in flight per lane (four from twelve chunks per lane on, with eight waves).  More in
  // flight per lane means fewer rows in flight per CU and measured 5-25 % slower.
  // (a row need not be a whole number of passes: K = 11008 and 18944 measured 7.8 and
  // 10.2 us with 32 lanes per row against 10.7 and 15.8 us with 16)
  // Fewer rows than give every CU two workgroups of four waves: more lanes per row (a
  // 1024 x 1024 matrix took 4.4 us with 16 lanes per row and 3.4 us with 64).
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  int lpr = nchunks > 128 ? 32 : 16;
  const bool long_at_base = (nchunks + lpr - 1) / lpr >= 12;  // long rows keep their lanes (K = 18944: 10.2 against 12.6 us)
  while (!long_at_base && lpr < 64 && p.n * lpr / 256 < 2 * cus) lpr *= 2;
  const int per_lane = (int)((nchunks + lpr - 1) / lpr);
  const bool long_rows = per_lane >= 12;
  // int8 (half the weights per chunk, half the arithmetic per byte loaded): four chunks in
  // flight from eight per lane on (4096..12288 x 4096 at M = 1, 2: 5.7-11.8 us against
  // 6.2-13.0 us with two, all three int8 formats)
  const bool int8_mid_rows = p.format != TLHIP_FMT_INT4_GROUPED && per_lane >= 8;
  return gemv_cfg(lpr, 1, long_rows ? 8 : 4, 1, long_rows || int8_mid_rows ? 4 : 2);
}

std::vector<tlhip_kernel_config_t> candidates(const Problem& p) {
  std::vector<tlhip_kernel_config_t> out;
  if (p.m <= 16) {
    for (int lpr : {16, 32, 64})
      for (int r : {1, 2, 4})
        for (int waves : {2, 4, 8})
          for (int kw : {1, 2, 4})
            for (int unroll : {2, 4, 8}) {
              if (kw > waves) continue;
              tlhip_kernel_config_t c = gemv_cfg(lpr, r, waves, kw, unroll);
              if (gemv_config_applicable(p, c, nullptr)) out.push_back(c);
            }
  }
  if (p.m <= 4) {
    // the 4x4x4 matrix-core form of the same kernel
    for (int waves : {2, 4, 8})
      for (int kw : {1, 2, 4})
        for (int unroll : {2, 4, 8}) {
          if (kw > waves) continue;
          tlhip_kernel_config_t c = gemv_cfg(16, 1, waves, kw, unroll);
          c.p5 = 1;
          if (gemv_config_applicable(p, c, nullptr)) out.push_back(c);
        }
  }
  if (p.m <= 64) {  // above 16 rows: two or four tiles of rows per weight row block
    for (int waves : {4, 8, 16})
      for (int unroll : {1, 2, 4})
        for (int kw : {1, 2, 4, 8, 16})
          for (int ks : {1, 2, 4, 8, 16}) {
            if (kw > waves) continue;
            tlhip_kernel_config_t c = mfma_cfg(waves, unroll, kw, ks);
            if (gemv_mfma_config_applicable(p, c, nullptr)) out.push_back(c);
            c.p5 = 1;  // whole-line weight loads
            if (gemv_mfma_config_applicable(p, c, nullptr)) out.push_back(c);
          }
  }
  if (p.m <= 16) {
    for (int waves : {4, 8, 16})
      for (int unroll : {1, 2})
        for (int per_cu : {1, 2})
          for (int ks : {1, 2, 4, 8, 16})
            for (int upfront : {0, 1})
              for (int xbar : {0, 1}) {
                tlhip_kernel_config_t c = xreg_cfg(waves, unroll, per_cu, ks, upfront, xbar);
                if (gemv_xreg_config_applicable(p, c, nullptr)) out.push_back(c);
              }
    for (int waves : {4, 8})
      for (int depth : {2, 3, 4})
        for (int per_cu : {1, 2})
          for (int unroll : {1, 2}) {
            tlhip_kernel_config_t c = wave_cfg(waves, depth, per_cu, unroll);
            if (gemv_wave_config_applicable(p, c, nullptr)) out.push_back(c);
            c.p5 = 1;  // whole-line weight loads
            if (gemv_wave_config_applicable(p, c, nullptr)) out.push_back(c);
          }
  }
  if (p.x_dtype == TLHIP_F16 && p.m >= 16) {
    static const int tiles[][5] = {
        {128, 128, 64, 2, 2}, {256, 128, 64, 2, 2}, {128, 256, 64, 2, 2},
        {256, 256, 64, 2, 2}, {64, 128, 64, 2, 2},
    };
    for (auto& t : tiles) {
      tlhip_kernel_config_t c = tiled_cfg(t[0], t[1], t[2], t[3], t[4]);
      if (gemm_config_applicable(p, c, nullptr)) out.push_back(c);
      // K slices across workgroups where the tiles are fewer than the CUs
      if (t[0] <= 128 && t[1] == 128 &&
          ((p.m + t[0] - 1) / t[0]) * ((p.n + t[1] - 1) / t[1]) < (device_cu_count() > 0 ? device_cu_count() : 256))
        for (int ks : {2, 4, 8}) {
          c.p5 = ks;
          if (gemm_config_applicable(p, c, nullptr)) out.push_back(c);
        }
    }
    static const int direct[][4] = {{256, 256, 2, 4}, {256, 128, 2, 4}, {128, 256, 2, 4}, {256, 128, 4, 2}, {128, 128, 2, 2}, {256, 256, 2, 2}, {128, 256, 1, 4}, {128, 192, 2, 2}};
    for (auto& t : direct) {
      tlhip_kernel_config_t c = direct_cfg(t[0], t[1], t[2], t[3]);
      if (gemm_direct_config_applicable(p, c, nullptr)) out.push_back(c);
    }
    // K slices across workgroups where the 128 x 128 tiles are fewer than the CUs
    if (((p.m + 127) / 128) * ((p.n + 127) / 128) < (device_cu_count() > 0 ? device_cu_count() : 256))
      for (int ks : {2, 4, 8})
        for (auto& t : {std::array<int, 4>{128, 128, 2, 2}, std::array<int, 4>{128, 256, 1, 4}}) {
          tlhip_kernel_config_t c = direct_cfg(t[0], t[1], t[2], t[3]);
          c.p5 = ks;
          if (gemm_direct_config_applicable(p, c, nullptr)) out.push_back(c);
        }
  }
  return out;
}

// Caller holds g_tune_mutex.
bool nearest_in_class(const Problem& p, const std::vector<ClassEntry>& list, tlhip_kernel_config_t* out) {
  double best = 1e30;
  bool found = false;
  for (const auto& e : list) {
    const double dn = std::fabs(std::log2((double)e.n / (double)p.n));
    const double dk = std::fabs(std::log2((double)e.k / (double)p.k));
    const double dm = std::fabs(std::log2((double)e.m / (double)p.m));
    if (dn > 1.0 || dk > 1.0 || dm > 1.0) continue;
    // Winners do not carry over to another row count.  Decode kernels are tuned to theirs
    // (the activations a workgroup stages and the registers a lane holds grow with it: the
    // LM head's M = 8 winner measured 150 us at M = 16 against 106 us for the heuristic default
    // at M = 16; a prefill winner is fitted to its number of tiles: the 256 x 128 tile
    // that wins M = 512 at 12288 x 4096 took 71 us at M = 256 against 54 us for the default)
    if (e.m != p.m) continue;
    const double d = dn + 2.0 * dk + dm;  // K decides whether the activations fit LDS: weigh it
    if (d < best && config_applicable(p, e.config, nullptr)) {
      best = d;
      *out = e.config;
      found = true;
    }
  }
  return found;
}

// The winner of the nearest tuned problem of the same class (autotune.ts:269-300's
// per-shape-class cache), re-gated on applicability.  "Near" = N and K each within a
// factor of two and the same number of rows;
// farther than that the hand heuristic knows more than a foreign winner does.
// The output type only changes the store at the end of a kernel, so where the class of
// p's own output type holds nothing near, the class of the other output type is asked.
bool class_config(const Problem& p, tlhip_kernel_config_t* out) {
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  Problem other = p;
  other.y_dtype = p.y_dtype == TLHIP_F16 ? TLHIP_F32 : TLHIP_F16;
  for (const Problem* asked : {&p, (const Problem*)&other}) {
    auto it = g_class_tuned.find(class_key(*asked));
    if (it == g_class_tuned.end()) continue;
    if (nearest_in_class(p, it->second, out)) return true;
  }
  return false;
}

tlhip_kernel_config_t select_config(const Problem& p) {
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    auto it = g_tuned.find(problem_key(p));
    if (it != g_tuned.end() && config_applicable(p, it->second, nullptr)) return it->second;
  }
  tlhip_kernel_config_t c;
  if (class_config(p, &c)) return c;
  return default_config(p);
}

// The VALU configuration for launches only that kernel has (grouped, with a prologue):
// the tuned or selected one if it is of that kernel, else the heuristic.
tlhip_kernel_config_t valu_config(const Problem& p) {
  tlhip_kernel_config_t c = select_config(p);
  if (c.variant != VARIANT_GEMV) c = default_valu_config(p);
  return c;
}

// The grouped kernel is the dot2 form with two chunks in flight and one or two rows
// per lane group: the tuned geometry where it is of that form, else the default one.
tlhip_kernel_config_t grouped_config(const Problem& p) {
  tlhip_kernel_config_t c = valu_config(p);
  if (c.p5 != 0) c = default_valu_config(p);
  c.p4 = 2;
  if (c.p1 > 2) c.p1 = 2;
  return c;
}

int run_config(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  if (c.variant == VARIANT_TILED_DIRECT) return launch_gemm_direct(p, c, stream);
  if (c.variant == VARIANT_TILED) return launch_gemm(p, c, stream);
  if (c.variant == VARIANT_GEMV_MFMA) return launch_gemv_mfma(p, c, stream);
  if (c.variant == VARIANT_GEMV_XREG) return launch_gemv_xreg(p, c, stream);
  if (c.variant == VARIANT_GEMV_WAVE) return launch_gemv_wave(p, c, stream);
  return launch_gemv(p, c, stream);
}

// From this many rows on, f32 activations take the matrix-core route below: up to 16 rows
// (decode) stay on the f32 arithmetic of the VALU kernel; beyond, that kernel would stream
// the weights once per four rows (63 rows: 16 times).
constexpr int64_t kF32TiledFromRows = 17;

// The problem an f32-activation prefill runs as: the same one on f16 activations.
Problem as_f16_activations(const Problem& p) {
  Problem q = p;
  q.x_dtype = TLHIP_F16;
  return q;
}

// f32 activations, many rows: the matrix cores take f16 operands, so the rows are
// rounded to f16 once (a cast launch into the stream's workspace, as many rows at a time
// as it holds) and go through the tiled kernel selected for the f16 problem.  Returns
// false when this route does not apply (no tiled kernel for the shape, K too long for
// the workspace) and nothing was launched.
bool f32_rows_through_tiled(const Problem& p, hipStream_t stream, int* rc) {
  if (p.x_dtype != TLHIP_F32 || p.m < kF32TiledFromRows || p.pro.kind != TLHIP_PRO_NONE) return false;
  Problem q = as_f16_activations(p);
  tlhip_kernel_config_t c = select_config(q);
  // (a tuned winner of the f16 problem may be the skinny kernel, which keeps its K-slice
  // tiles where the rounded rows are: the heuristic tile then)
  if (c.variant != VARIANT_TILED && c.variant != VARIANT_TILED_DIRECT) c = default_config(q);
  if (c.variant != VARIANT_TILED && c.variant != VARIANT_TILED_DIRECT) return false;
  c.p5 = 0;  // no K split across workgroups: its partial sums live in the workspace too
  const int64_t capacity = (int64_t)(kSplitWorkspaceFloats * sizeof(float) / sizeof(_Float16));
  int64_t rows = capacity / std::max<int64_t>(p.k, 1);
  if (rows >= 256) rows -= rows % 256;  // whole tiles per chunk
  if (rows < 32) return false;
  float* workspace = nullptr;
  int* counters = nullptr;
  *rc = split_workspace(stream, &workspace, &counters);
  if (*rc) return true;
  const int yb = p.y_dtype == TLHIP_F16 ? 2 : 4;
  for (int64_t m0 = 0; m0 < p.m; m0 += rows) {
    q.m = std::min<int64_t>(rows, p.m - m0);
    *rc = tlhip_cast((const float*)p.x + m0 * p.k, TLHIP_F32, workspace, TLHIP_F16, q.m * p.k, (tlhip_stream_t)stream);
    if (*rc) return true;
    q.x = workspace;
    q.y = (char*)p.y + m0 * p.n * yb;
    q.epi = epilogue_from_row(p.epi, m0, p.n);
    *rc = run_config(q, c, stream);
    if (*rc) return true;
  }
  return true;
}

int matmul_with(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  if (c.variant == VARIANT_TILED || c.variant == VARIANT_TILED_DIRECT) return run_config(p, c, stream);
  if (p.m <= 16) return run_config(p, c, stream);
  // 17..64 rows in one launch of the skinny matrix-core kernel (two or four tiles of 16 rows)
  if (p.m <= 64 && c.variant == VARIANT_GEMV_MFMA && gemv_mfma_config_applicable(p, c, nullptr)) return run_config(p, c, stream);
  int rc = TLHIP_OK;
  if (f32_rows_through_tiled(p, stream, &rc)) return rc;
  // f32 activations below kF32TiledFromRows rows (or a shape the tiled kernels reject):
  // GEMV passes of 16 rows.  Declared, slow: every pass streams the weights again.
  const int xb = p.x_dtype == TLHIP_F16 ? 2 : 4, yb = p.y_dtype == TLHIP_F16 ? 2 : 4;
  for (int64_t m0 = 0; m0 < p.m; m0 += 16) {
    Problem q = p;
    q.m = std::min<int64_t>(16, p.m - m0);
    q.x = (const char*)p.x + m0 * p.k * xb;
    q.y = (char*)p.y + m0 * p.n * yb;
    q.epi = epilogue_from_row(p.epi, m0, p.n);
    int rc = run_config(q, c, stream);
    if (rc) return rc;
  }
  return TLHIP_OK;
}

// 17..64 rows in ONE launch of the skinny matrix-core kernel: eight waves, two iterations
// in flight, the fewest K slices across workgroups whose activations fit LDS, and the
// fewest K-split waves per row block that still give every CU a workgroup (measured best
// or within 5 % of it at 4096..28672 x 4096..12288, M = 24..64).
bool rows_in_one_launch_config(const Problem& p, tlhip_kernel_config_t* out) {
  if (p.m <= 16 || p.m > 64 || p.x_dtype != TLHIP_F16) return false;
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  const int64_t nblocks = (p.n + 15) / 16;
  for (int ks = 1; ks <= 16; ks *= 2) {
    int fill = 1;  // K-split waves per row block: 8 / fill row blocks per workgroup
    while (fill < 8 && (nblocks * fill / 8) * ks < cus) fill *= 2;
    for (int kw : {fill, 8, 4, 2, 1})
      for (int unroll : {2, 1}) {
        const tlhip_kernel_config_t c = mfma_cfg(8, unroll, kw, ks);
        if (gemv_mfma_config_applicable(p, c, nullptr)) {
          *out = c;
          return true;
        }
      }
  }
  return false;
}

bool has_tuned_entry(const Problem& p) {
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  return g_tuned.count(problem_key(p)) != 0;
}

// What the library launches for a problem when the caller names no configuration: the
// selected configuration on all rows, or the rows in chunks.
struct Route {
  int64_t chunk;                // rows per launch; 0: one launch (or matmul_with's own passes) of `first` on all rows
  tlhip_kernel_config_t first;  // configuration of the whole chunks (of everything when chunk == 0)
  tlhip_kernel_config_t last;   // configuration of the remaining rows, if any
};

// 9..16 rows whose activations fit no geometry of the matrix-core kernels (a very long K
// whose steps no power of two up to 16 slices finely enough) would fall to the VALU kernel,
// which streams the weights once per four rows; two launches of at most 8 rows on the
// matrix cores stream them twice.  (K = 11008 and 13696 were such cases until the kernel
// took K slices of unequal length.)
//
// A few more rows than the decode kernels take, far fewer than fill the chip with
// tiles: a tiled launch of at most one round of 128 x 128 tiles takes the time ONE
// workgroup needs to walk K (measured 40-45 us per 4096 of K whatever M and N are, up
// to 512 resident tiles), the decode kernel streams the weights once per 16 rows (3 us
// + 1 us per 3.2 MB of packed weights: 6.3 / 9.9 / 11.9 us at the Qwen3-8B shapes).
// Below the break-even the rows go through the decode kernel: up to 64 per launch, or
// 16 at a time where the activations of more rows fit no geometry.
// (A tuned entry of the problem itself is a measurement and stands.)
Route plan_route(const Problem& p, const tlhip_kernel_config_t& c) {
  Route r{0, c, c};
  if (p.pro.kind != TLHIP_PRO_NONE) return r;
  if (c.variant == VARIANT_GEMV && p.m > 8 && p.m <= 16) {
    Problem lo = p, hi = p;
    lo.m = 8;
    hi.m = p.m - 8;
    const tlhip_kernel_config_t cl = select_config(lo);
    if (cl.variant == VARIANT_GEMV_MFMA || cl.variant == VARIANT_GEMV_XREG) return Route{8, cl, select_gemv_config(hi)};
    return r;
  }
  if ((c.variant == VARIANT_TILED || c.variant == VARIANT_TILED_DIRECT) && p.m > 16 && p.x_dtype == TLHIP_F16 &&
      !has_tuned_entry(p)) {
    const double packed_mb = (double)p.n * (double)p.k * (p.format == TLHIP_FMT_INT4_GROUPED ? 0.5 : 1.0) / 1e6;
    const double pass_us = g_model.pass_base_us + packed_mb / g_model.pass_mb_per_us;
    const int64_t passes = (p.m + 15) / 16;
    const int64_t tiles = ((p.m + 127) / 128) * ((p.n + 127) / 128);
    const double rounds = (double)tiles <= g_model.resident_tiles ? 1.0 : (double)tiles / g_model.resident_tiles;
    const double tiled_us =
        direct_round_us(p, c.p5 > 1 ? c.p5 : 1,
                        c.variant == VARIANT_TILED_DIRECT ? g_model.walk_direct_us
                                                          : (c.p0 <= 64 ? g_model.walk_staged64_us : g_model.walk_staged128_us)) *
        rounds;
    // Up to 64 rows per launch of the decode kernel: 1.2-1.6 times a 16-row pass for two
    // tiles of rows, 2.3-3.2 times for four (the activations a workgroup stages grow with
    // the rows, and their K slices are combined across workgroups).  More rows go 64 at a
    // time while that beats the tiles (128 rows at 4096 x 4096: 2 x 16 us against 49 us).
    auto chunk_us = [&](int64_t rows) { return pass_us * (rows <= 16 ? 1.0 : (rows <= 32 ? g_model.rows32_factor : g_model.rows64_factor)); };
    const int64_t full = p.m / 64, rest = p.m % 64;
    const double rows_us = (double)full * chunk_us(64) + (rest ? chunk_us(rest) : 0.0);
    if (rows_us < g_model.rows_break_even * tiled_us) {
      bool ok = true;
      Route q{64, c, c};
      Problem q64 = p, qr = p;
      q64.m = 64;
      qr.m = rest;
      if (full) ok = rows_in_one_launch_config(q64, &q.first);
      if (ok && rest > 16) ok = rows_in_one_launch_config(qr, &q.last);
      if (ok && rest > 0 && rest <= 16) {
        q.last = select_gemv_config(qr);
        ok = q.last.variant == VARIANT_GEMV_MFMA || q.last.variant == VARIANT_GEMV_XREG || rest <= 4;
      }
      if (!full) q.first = q.last;
      if (ok) return q;
    }
    if ((double)passes * pass_us < g_model.passes_break_even * tiled_us) {
      Problem q = p;
      q.m = 16;
      const tlhip_kernel_config_t c16 = select_gemv_config(q);
      if (c16.variant == VARIANT_GEMV_MFMA || c16.variant == VARIANT_GEMV_XREG) return Route{0, c16, c16};  // matmul_with's passes
    }
  }
  return r;
}

// The first step of the chain that runs behind the GEMM in a launch of its own, or -1.  In
// a GEMM's own epilogue a binary step reads its [M,N] input in the accumulators' layout,
// a chain per element; on a large output one pass over the finished rows, 16 bytes a lane,
// costs less than that (2048 x 12288, bias + silu + add: 359 us fused).  The steps before
// the binary one stay fused; an f16 output is rounded to f16 between the two launches.
int epilogue_tail_from(const Problem& p) {
  if (p.m <= 64 || (double)p.m * (double)p.n < g_model.binary_tail_elements) return -1;
  if (!epilogue_tail_applicable(p.y, p.n)) return -1;
  for (int i = 0; i < p.epi.n_ops; ++i)
    if (p.epi.kind[i] == TLHIP_EPI_BINARY) return i;
  return -1;
}

int run_selected(const Problem& p0, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const int tail_from = epilogue_tail_from(p0);
  if (tail_from >= 0) {
    Problem head = p0;
    head.epi.n_ops = tail_from;
    int rc = run_selected(head, c, stream);
    if (rc) return rc;
    DevEpilogue tail;
    memset(&tail, 0, sizeof tail);
    for (int i = tail_from; i < p0.epi.n_ops; ++i) {
      const int j = tail.n_ops++;
      tail.kind[j] = p0.epi.kind[i];
      tail.unary[j] = p0.epi.unary[i];
      tail.input_dtype[j] = p0.epi.input_dtype[i];
      tail.input[j] = p0.epi.input[i];
    }
    return launch_epilogue_tail(p0.y, p0.y_dtype, p0.m, p0.n, tail, stream);
  }
  const Problem& p = p0;
  const Route r = plan_route(p, c);
  if (r.chunk == 0) return matmul_with(p, r.first, stream);
  const int xb = p.x_dtype == TLHIP_F16 ? 2 : 4, yb = p.y_dtype == TLHIP_F16 ? 2 : 4;
  for (int64_t m0 = 0; m0 < p.m; m0 += r.chunk) {
    Problem q = p;
    q.m = std::min<int64_t>(r.chunk, p.m - m0);
    q.x = (const char*)p.x + m0 * p.k * xb;
    q.y = (char*)p.y + m0 * p.n * yb;
    q.epi = epilogue_from_row(p.epi, m0, p.n);
    const int rc = matmul_with(q, q.m == r.chunk ? r.first : r.last, stream);
    if (rc) return rc;
  }
  return TLHIP_OK;
}

// One-field variations of `base` inside its kernel family, plus the heuristic defaults of
// the families: the quick search of generateNeighborConfigs (autotune.ts:419-465).
std::vector<tlhip_kernel_config_t> neighbour_candidates(const Problem& p, const tlhip_kernel_config_t& base) {
  std::vector<tlhip_kernel_config_t> out;
  auto same = [](const tlhip_kernel_config_t& a, const tlhip_kernel_config_t& b) { return !memcmp(&a, &b, sizeof a); };
  auto push = [&](const tlhip_kernel_config_t& c) {
    if (!config_applicable(p, c, nullptr)) return;
    for (const auto& o : out)
      if (same(o, c)) return;
    out.push_back(c);
  };
  push(base);
  auto vary = [&](int field, std::initializer_list<int> values) {
    for (int v : values) {
      tlhip_kernel_config_t c = base;
      (&c.p0)[field] = v;
      push(c);
    }
  };
  switch (base.variant) {
    case VARIANT_GEMV:
      vary(0, {16, 32, 64});
      vary(1, {1, 2, 4});
      vary(2, {2, 4, 8});
      vary(3, {1, 2, 4});
      vary(4, {2, 4, 8});
      vary(5, {0, 1});
      break;
    case VARIANT_GEMV_MFMA:
      vary(0, {4, 8, 16});
      vary(1, {1, 2, 4});
      vary(2, {1, 2, 4, 8, 16});
      vary(3, {1, 2, 4, 8});
      vary(5, {0, 1});
      break;
    case VARIANT_GEMV_WAVE:
      vary(0, {4, 8});
      vary(1, {2, 3, 4});
      vary(2, {1, 2});
      vary(3, {1, 2});
      vary(5, {0, 1});
      break;
    case VARIANT_GEMV_XREG:
      vary(0, {4, 8, 16});
      vary(1, {1, 2});
      vary(2, {1, 2});
      vary(3, {1, 2, 4, 8, 16});
      vary(4, {0, 1});
      vary(5, {0, 1});
      break;
    default:
      for (const auto& c : candidates(p))
        if (c.variant == VARIANT_TILED || c.variant == VARIANT_TILED_DIRECT) push(c);
      break;
  }
  push(default_config(p));
  if (p.m <= 16) push(default_valu_config(p));
  return out;
}

struct TuneOptions {
  int reps = 0;           // launches per event pair; 0 = sized so that a batch takes about 300 us (20..100)
  int batches = 3;        // timed batches per candidate, median (dispatch.ts:324-397: 3 timed runs)
  int retime_top = 3;     // the fastest candidates timed once more, three times as long, minimum
  double warm_ms = 30.0;  // GPU milliseconds of untimed launches first: the clock ramps up after a pause
  bool quick = false;     // neighbours of the current choice instead of every candidate
  size_t pool_bytes = (size_t)640 << 20;  // alias copies of the weight the tuner makes when given only one buffer
};

struct WeightAlias {
  const void* packed;
  const void* scales;
};

size_t packed_bytes(const Problem& p) { return (size_t)p.n * (size_t)p.k / (p.format == TLHIP_FMT_INT4_GROUPED ? 2 : 1); }
size_t scales_bytes(const Problem& p) {
  return p.format == TLHIP_FMT_INT8_ROW ? (size_t)p.n * 4 : (size_t)p.n * (size_t)(p.k / p.group_size) * 2;
}

// Times the candidates for `p` and caches the winner.  `aliases`: the weight in distinct
// buffers (same contents or not, same shape), rotated launch by launch so that a weight
// smaller than the 256 MB last-level cache is still timed from HBM; with a single
// buffer the tuner makes its own copies, up to `pool_bytes`, and frees them afterwards.
int autotune_problem(const Problem& p0, std::vector<WeightAlias> aliases, const TuneOptions& o, hipStream_t stream,
                     double* best_us_out) {
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    if (g_autotuning) return TLHIP_OK;
  }
  hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &cap) == hipSuccess && cap != hipStreamCaptureStatusNone) return TLHIP_OK;
  std::lock_guard<std::mutex> run_lock(g_tune_run_mutex);
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    g_autotuning = true;
  }
  struct Done {
    ~Done() {
      std::lock_guard<std::mutex> lock(g_tune_mutex);
      g_autotuning = false;
    }
  } done;

  if (aliases.empty()) aliases.push_back({p0.packed, p0.scales});
  std::vector<void*> owned;
  struct FreeOwned {
    std::vector<void*>& v;
    hipStream_t s;
    ~FreeOwned() {
      if (v.empty()) return;
      (void)hipStreamSynchronize(s);
      for (void* q : v) (void)hipFree(q);
    }
  } free_owned{owned, stream};
  const size_t pb = packed_bytes(p0), sb = scales_bytes(p0);
  if (aliases.size() == 1 && o.pool_bytes > pb + sb && pb + sb < ((size_t)256 << 20)) {
    size_t want = o.pool_bytes / (pb + sb);
    if (want > 95) want = 95;
    for (size_t i = 0; i < want; ++i) {
      void *wp = nullptr, *sp = nullptr;
      if (hipMalloc(&wp, pb) != hipSuccess) break;
      if (hipMalloc(&sp, sb) != hipSuccess) {
        (void)hipFree(wp);
        break;
      }
      owned.push_back(wp);
      owned.push_back(sp);
      if (hipMemcpyAsync(wp, p0.packed, pb, hipMemcpyDeviceToDevice, stream) != hipSuccess ||
          hipMemcpyAsync(sp, p0.scales, sb, hipMemcpyDeviceToDevice, stream) != hipSuccess)
        break;
      aliases.push_back({wp, sp});
    }
    (void)hipGetLastError();  // a failed allocation only means fewer aliases
  }

  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess) return set_error(TLHIP_ERR_DEVICE, "autotune: hipEventCreate failed");
  if (hipEventCreate(&e1) != hipSuccess) {
    (void)hipEventDestroy(e0);
    return set_error(TLHIP_ERR_DEVICE, "autotune: hipEventCreate failed");
  }
  struct FreeEvents {
    hipEvent_t a, b;
    ~FreeEvents() {
      (void)hipEventDestroy(a);
      (void)hipEventDestroy(b);
    }
  } free_events{e0, e1};

  size_t turn = 0;
  auto launch = [&](const tlhip_kernel_config_t& c) {
    Problem q = p0;
    const WeightAlias& a = aliases[turn++ % aliases.size()];
    q.packed = a.packed;
    q.scales = a.scales;
    return matmul_with(q, c, stream) == TLHIP_OK;
  };
  // microseconds per launch of `reps` back-to-back launches; < 0: the candidate failed
  int device_error = 0;
  auto time_batch = [&](const tlhip_kernel_config_t& c, int reps) -> double {
    if (hipEventRecord(e0, stream) != hipSuccess) return -1.0;
    for (int i = 0; i < reps; ++i)
      if (!launch(c)) {
        (void)hipStreamSynchronize(stream);
        return -1.0;
      }
    if (hipEventRecord(e1, stream) != hipSuccess || hipEventSynchronize(e1) != hipSuccess) {
      device_error = 1;
      return -1.0;
    }
    float ms = 0;
    (void)hipEventElapsedTime(&ms, e0, e1);
    return (double)ms * 1000.0 / reps;
  };

  const tlhip_kernel_config_t current = select_config(p0);
  // warm-up on the current choice, and the batch length from its time
  double cur_us = time_batch(current, 20);
  if (device_error) return set_error(TLHIP_ERR_DEVICE, "autotune: a timing event failed");
  if (cur_us <= 0) cur_us = 10.0;
  int reps = o.reps > 0 ? o.reps : (int)(300.0 / cur_us);
  if (o.reps <= 0) reps = reps < 20 ? 20 : (reps > 100 ? 100 : reps);
  for (double spent = 0; spent < o.warm_ms * 1e3;) {
    const double us = time_batch(current, reps);
    if (us <= 0) break;
    spent += us * reps;
  }

  const std::vector<tlhip_kernel_config_t> cands = o.quick ? neighbour_candidates(p0, current) : candidates(p0);
  std::vector<std::pair<double, tlhip_kernel_config_t>> timed;
  const int batches = o.batches < 1 ? 1 : (o.batches > 9 ? 9 : o.batches);
  for (const auto& c : cands) {
    if (!launch(c) || !launch(c)) {  // two untimed launches (dispatch.ts:324-397: 2 warm-up runs)
      (void)hipStreamSynchronize(stream);
      continue;
    }
    double t[9];
    bool ok = true;
    for (int i = 0; i < batches && ok; ++i) {
      t[i] = time_batch(c, reps);
      ok = t[i] > 0;
    }
    if (device_error) return set_error(TLHIP_ERR_DEVICE, "autotune: a timing event failed");
    if (!ok) continue;
    std::sort(t, t + batches);
    timed.push_back({t[batches / 2], c});
  }
  if (timed.empty()) return set_error(TLHIP_ERR_INVALID, "autotune: no candidate configuration ran for %s", problem_key(p0).c_str());
  std::sort(timed.begin(), timed.end(), [](const auto& a, const auto& b) { return a.first < b.first; });
  double best = timed[0].first;
  tlhip_kernel_config_t best_cfg = timed[0].second;
  // candidates within a few per cent of each other change places from run to run: the
  // fastest few once more, three times as long, the minimum of three batches
  if (o.retime_top > 1 && timed.size() > 1) {
    best = 1e30;
    const size_t top = std::min<size_t>(timed.size(), (size_t)o.retime_top);
    for (size_t i = 0; i < top; ++i) {
      double us = 1e30;
      for (int r = 0; r < 3; ++r) {
        const double v = time_batch(timed[i].second, 3 * reps);
        if (v > 0 && v < us) us = v;
      }
      if (device_error) return set_error(TLHIP_ERR_DEVICE, "autotune: a timing event failed");
      if (us < best) {
        best = us;
        best_cfg = timed[i].second;
      }
    }
  }
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    record_winner_locked(p0, best_cfg);
  }
  count_autotune_run();
  if (best_us_out) *best_us_out = best;
  if (getenv("TORCHLETTE_DEBUG_AUTOTUNE"))
    fprintf(stderr, "[tlhip autotune] %s: %zu candidates, %zu weight buffers, %d launches per batch -> variant %d "
                    "(%d,%d,%d,%d,%d,%d) %.2f us\n",
            problem_key(p0).c_str(), cands.size(), aliases.size(), reps, best_cfg.variant, best_cfg.p0, best_cfg.p1,
            best_cfg.p2, best_cfg.p3, best_cfg.p4, best_cfg.p5, best);
  return TLHIP_OK;
}

}  // namespace

tlhip_kernel_config_t select_gemv_config(const Problem& p) {
  tlhip_kernel_config_t c = select_config(p);
  if (c.variant == VARIANT_TILED || c.variant == VARIANT_TILED_DIRECT) c = default_config(p);
  return c;
}

int run_kernel_config(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) { return run_config(p, c, stream); }

// What tlhip_gemv runs for `p` (the selected configuration and its route: one launch, rows
// in chunks, or passes), for an entry point that brings its own scratch in p.scratch; and
// the most K slices any launch of that route takes (1: the route needs no scratch).
int run_gemv_route(const Problem& p, hipStream_t stream) { return run_selected(p, select_gemv_config(p), stream); }
int gemv_route_k_slices(const Problem& p) {
  const Route r = plan_route(p, select_gemv_config(p));
  const int first = config_k_slices(r.first);
  return r.chunk == 0 ? first : std::max(first, config_k_slices(r.last));
}

// The tuning file that ships next to the library: <directory of libtlhip.so>/tuning/
// mi355x.json, or the file TLHIP_TUNING_FILE names ("none" = load nothing).  Called by
// tlhip_init, so every binding gets the committed winners, not only the benchmark.
// A missing or malformed file is not an error: the heuristic defaults serve.
int load_default_tuning() {
  std::string path;
  if (const char* e = getenv("TLHIP_TUNING_FILE")) {
    if (!strcmp(e, "none") || !*e) return 0;
    path = e;
  } else {
    Dl_info info;
    if (!dladdr((const void*)&load_default_tuning, &info) || !info.dli_fname) return 0;
    path = info.dli_fname;
    const size_t slash = path.rfind('/');
    path = (slash == std::string::npos ? std::string(".") : path.substr(0, slash)) + "/tuning/mi355x.json";
  }
  FILE* f = fopen(path.c_str(), "rb");
  if (!f) return 0;
  std::string text;
  char buf[4096];
  size_t got;
  while ((got = fread(buf, 1, sizeof buf, f)) > 0) text.append(buf, got);
  fclose(f);
  size_t before;
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    before = g_tuned.size();
  }
  if (tlhip_tune_cache_import(text.c_str()) != TLHIP_OK) {
    if (getenv("TORCHLETTE_DEBUG_AUTOTUNE")) fprintf(stderr, "[tlhip] tuning file %s ignored: %s\n", path.c_str(), tlhip_last_error());
    clear_error();
    return 0;
  }
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  return (int)(g_tuned.size() - before);
}

int config_k_slices(const tlhip_kernel_config_t& c) {
  if (c.variant == VARIANT_GEMV_MFMA || c.variant == VARIANT_GEMV_XREG) return c.p3 < 1 ? 1 : c.p3;
  return 1;
}

int validate_weight(const tlhip_qweight_t* w, const char* who) {
  if (!w) return set_error(TLHIP_ERR_INVALID, "%s: missing packing/scales on B operand", who);
  if (w->format != TLHIP_FMT_INT8_GROUPED && w->format != TLHIP_FMT_INT8_ROW &&
      w->format != TLHIP_FMT_INT4_GROUPED)
    return set_error(TLHIP_ERR_INVALID, "%s: unsupported scheme %d", who, w->format);
  if (w->n < 0 || w->k < 0) return set_error(TLHIP_ERR_INVALID, "%s: negative shape", who);
  if (w->n > 0 && w->k > 0 && (!w->packed || !w->scales))
    return set_error(TLHIP_ERR_INVALID, "%s: missing packing/scales on B operand", who);
  const int per_word = w->format == TLHIP_FMT_INT4_GROUPED ? 8 : 4;
  if (w->k % per_word != 0)
    return set_error(TLHIP_ERR_INVALID, "%s: K=%lld must be divisible by %d", who, (long long)w->k, per_word);
  if (w->format != TLHIP_FMT_INT8_ROW) {
    if (w->group_size <= 0 || !is_pow2(w->group_size))
      return set_error(TLHIP_ERR_INVALID, "%s: groupSize %d must be a power of two", who, w->group_size);
    if (w->k % w->group_size != 0)
      return set_error(TLHIP_ERR_INVALID, "%s: K=%lld must be divisible by groupSize=%d", who,
                       (long long)w->k, w->group_size);
  }
  if (w->k > (int64_t)1 << 24 || w->n > (int64_t)1 << 30)
    return set_error(TLHIP_ERR_INVALID, "%s: shape [%lld,%lld] exceeds the supported range", who,
                     (long long)w->n, (long long)w->k);
  if (((uintptr_t)w->packed & 15) != 0)
    return set_error(TLHIP_ERR_INVALID, "%s: packed weights must be 16-byte aligned", who);
  // the kernels load the scales of consecutive groups as 4-, 8- and 16-byte vectors
  if (((uintptr_t)w->scales & 15) != 0)
    return set_error(TLHIP_ERR_INVALID, "%s: scales must be 16-byte aligned", who);
  return TLHIP_OK;
}

// The epilogue of a call with m activation rows on weight w: kinds, ops, types, and that
// every input has the shape its step indexes it by.
int check_epilogue(const tlhip_qweight_t* w, int64_t m, const tlhip_epilogue_t* epilogue, const char* who) {
  if (epilogue->n_ops < 0 || epilogue->n_ops > TLHIP_MAX_EPILOGUE_OPS)
    return set_error(TLHIP_ERR_INVALID, "%s: epilogue has %d ops (max %d)", who, epilogue->n_ops, TLHIP_MAX_EPILOGUE_OPS);
  for (int i = 0; i < epilogue->n_ops; ++i) {
    const tlhip_epilogue_op_t& op = epilogue->ops[i];
    if (op.kind < TLHIP_EPI_NONE || op.kind > TLHIP_EPI_CAST_F16)
      return set_error(TLHIP_ERR_INVALID, "%s: unknown epilogue op kind %d", who, op.kind);
    if (op.kind == TLHIP_EPI_BINARY) {
      if (!op.input && w->n > 0 && m > 0) return set_error(TLHIP_ERR_INVALID, "%s: binary epilogue without input", who);
      if (op.input_dtype != TLHIP_F32 && op.input_dtype != TLHIP_F16)
        return set_error(TLHIP_ERR_INVALID, "%s: bad binary epilogue input dtype %d", who, op.input_dtype);
      if (op.unary < TLHIP_BINARY_ADD || op.unary > TLHIP_BINARY_MUL)
        return set_error(TLHIP_ERR_INVALID, "%s: unknown binary epilogue op %d (add, sub, mul)", who, op.unary);
      if ((int64_t)op.rows != m)
        return set_error(TLHIP_ERR_INVALID, "%s: a binary epilogue input must be [M,N] = [%lld,%lld]; its rows field says %d", who,
                         (long long)m, (long long)w->n, op.rows);
    }
    if (op.kind == TLHIP_EPI_BIAS) {
      if (!op.input && w->n > 0) return set_error(TLHIP_ERR_INVALID, "%s: bias epilogue without input", who);
      if (op.input_dtype != TLHIP_F32 && op.input_dtype != TLHIP_F16)
        return set_error(TLHIP_ERR_INVALID, "%s: bad bias dtype %d", who, op.input_dtype);
      if (op.rows != 1)
        return set_error(TLHIP_ERR_INVALID, "%s: a bias epilogue input must be [N] = [%lld]; its rows field says %d", who,
                         (long long)w->n, op.rows);
    }
    if (op.kind == TLHIP_EPI_UNARY && (op.unary < TLHIP_UNARY_NONE || op.unary > TLHIP_UNARY_TANH))
      return set_error(TLHIP_ERR_INVALID, "%s: unknown unary op %d", who, op.unary);
  }
  return TLHIP_OK;
}

int make_problem(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y, int y_dtype,
                 float alpha, const tlhip_epilogue_t* epilogue, Problem* p, const char* who) {
  int rc = validate_weight(w, who);
  if (rc) return rc;
  if (m < 0) return set_error(TLHIP_ERR_INVALID, "%s: negative M", who);
  if (x_dtype != TLHIP_F32 && x_dtype != TLHIP_F16) return set_error(TLHIP_ERR_INVALID, "%s: bad x dtype %d", who, x_dtype);
  if (y_dtype != TLHIP_F32 && y_dtype != TLHIP_F16) return set_error(TLHIP_ERR_INVALID, "%s: bad y dtype %d", who, y_dtype);
  if (m > 0 && w->k > 0 && !x) return set_error(TLHIP_ERR_INVALID, "%s: null activations", who);
  if (m > 0 && w->n > 0 && !y) return set_error(TLHIP_ERR_INVALID, "%s: null output", who);
  if (((uintptr_t)x & 15) != 0) return set_error(TLHIP_ERR_INVALID, "%s: activations must be 16-byte aligned", who);
  p->format = w->format;
  p->group_size = w->group_size;
  p->n = w->n;
  p->k = w->k;
  p->m = m;
  p->packed = w->packed;
  p->scales = w->scales;
  p->x = x;
  p->x_dtype = x_dtype;
  p->y = y;
  p->y_dtype = y_dtype;
  p->alpha = alpha;
  memset(&p->epi, 0, sizeof p->epi);
  memset(&p->pro, 0, sizeof p->pro);
  p->scratch = nullptr;
  if (epilogue) {
    const int rc = check_epilogue(w, m, epilogue, who);
    if (rc) return rc;
    p->epi.n_ops = epilogue->n_ops;
    for (int i = 0; i < epilogue->n_ops; ++i) {
      const tlhip_epilogue_op_t& op = epilogue->ops[i];
      p->epi.kind[i] = op.kind;
      p->epi.unary[i] = op.unary;
      p->epi.input[i] = op.input;
      p->epi.input_dtype[i] = op.input_dtype;
    }
  }
  return TLHIP_OK;
}

}  // namespace tlhip

using namespace tlhip;

extern "C" {

int tlhip_epilogue_check(const tlhip_qweight_t* w, int64_t m, const tlhip_epilogue_t* epilogue) {
  clear_error();
  if (!w) return set_error(TLHIP_ERR_INVALID, "epilogue_check: null weight");
  if (m < 0) return set_error(TLHIP_ERR_INVALID, "epilogue_check: negative m");
  return epilogue ? check_epilogue(w, m, epilogue, "epilogue_check") : TLHIP_OK;
}

int tlhip_dequant(const tlhip_qweight_t* w, float* out, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  int rc = validate_weight(w, "dequant");
  if (rc) return rc;
  if (w->n > 0 && w->k > 0 && !out) return set_error(TLHIP_ERR_INVALID, "dequant: null output");
  if (((uintptr_t)out & 15) != 0) return set_error(TLHIP_ERR_INVALID, "dequant: output must be 16-byte aligned");
  return launch_dequant(*w, out, resolve_stream(stream));
}

int tlhip_gemv(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y, int y_dtype,
               float alpha, const tlhip_epilogue_t* epilogue, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  Problem p;
  int rc = make_problem(w, x, x_dtype, m, y, y_dtype, alpha, epilogue, &p, "gemv");
  if (rc) return rc;
  if (m > 16) return set_error(TLHIP_ERR_INVALID, "gemv: M=%lld above 16; use tlhip_gemm_prefill", (long long)m);
  return run_selected(p, select_gemv_config(p), resolve_stream(stream));
}

int tlhip_gemv_grouped(const tlhip_gemv_problem_t* problems, int count, int x_dtype, int y_dtype, float alpha,
                       tlhip_stream_t stream) {
  return tlhip_gemv_grouped_rows(problems, count, x_dtype, 1, y_dtype, alpha, stream);
}

int tlhip_gemv_grouped_rows(const tlhip_gemv_problem_t* problems, int count, int x_dtype, int64_t m, int y_dtype,
                            float alpha, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (count < 0 || (count > 0 && !problems)) return set_error(TLHIP_ERR_INVALID, "gemv_grouped: bad problem list");
  if (count > 4) return set_error(TLHIP_ERR_INVALID, "gemv_grouped: a group holds at most 4 problems, got %d", count);
  if (m < 0 || m > 16) return set_error(TLHIP_ERR_INVALID, "gemv_grouped: M=%lld outside 0..16", (long long)m);
  Problem ps[4];
  for (int i = 0; i < count; ++i) {
    int rc = make_problem(&problems[i].w, problems[i].x, x_dtype, m, problems[i].y, y_dtype, alpha,
                          problems[i].epilogue, &ps[i], "gemv_grouped");
    if (rc) return rc;
  }
  if (count == 0 || m == 0) return TLHIP_OK;
  hipStream_t s = resolve_stream(stream);
  if (m == 1 && count > 1) {
    // one activation row: the configuration of the largest problem, in the VALU kernel's
    // grouped form (one grouped launch beats separate launches of whichever kernel is
    // fastest for a single problem: every launch costs 2-3 us)
    int big = 0;
    for (int i = 1; i < count; ++i)
      if (ps[i].n > ps[big].n) big = i;
    const tlhip_kernel_config_t c = grouped_config(ps[big]);
    if (gemv_group_compatible(ps, count, c, nullptr)) return launch_gemv_grouped(ps, count, c, s);
  }
  if (count > 1) {
    // Problems on the SAME activations (q/k/v, gate/up): one launch of a matrix-core
    // kernel, chosen as for one problem with all the rows (its tuned winner, or the winner
    // of the nearest tuned problem of its class).
    bool shared = true;
    int64_t rows = 0;
    for (int i = 0; i < count; ++i) {
      shared = shared && ps[i].x == ps[0].x && ps[i].k == ps[0].k;
      rows += ps[i].n;
    }
    if (shared && rows > 0) {
      Problem all = ps[0];
      all.n = rows;
      // ... and where that choice has no grouped form (the VALU kernel at several rows,
      // the per-wave pipelined kernel), the heuristic default of the same problem: one
      // launch of a slightly slower kernel beats `count` launches of the fastest one
      const tlhip_kernel_config_t tries[2] = {select_config(all), default_config(all)};
      for (const tlhip_kernel_config_t& c : tries) {
        if (c.variant == VARIANT_GEMV_MFMA && gemv_mfma_group_applicable(ps, count, c, nullptr))
          return launch_gemv_mfma_group(ps, count, c, s);
        if (c.variant == VARIANT_GEMV_XREG && gemv_xreg_group_applicable(ps, count, c, nullptr))
          return launch_gemv_xreg_group(ps, count, c, s);
      }
    }
  }
  for (int i = 0; i < count; ++i) {
    int rc = run_selected(ps[i], select_gemv_config(ps[i]), s);
    if (rc) return rc;
  }
  return TLHIP_OK;
}

// Checks a prologue against the problem it feeds and copies it into `p`.
static int attach_prologue(const tlhip_prologue_t* pro, Problem* p, const char* who) {
  if (!pro || pro->kind == TLHIP_PRO_NONE) return TLHIP_OK;
  if (pro->kind != TLHIP_PRO_RMSNORM && pro->kind != TLHIP_PRO_GATED_MUL)
    return set_error(TLHIP_ERR_INVALID, "%s: unknown prologue kind %d", who, pro->kind);
  if (!pro->operand && p->m > 0 && p->k > 0) return set_error(TLHIP_ERR_INVALID, "%s: prologue without operand", who);
  if (((uintptr_t)pro->operand & 15) != 0)
    return set_error(TLHIP_ERR_INVALID, "%s: prologue operand must be 16-byte aligned", who);
  if (pro->kind == TLHIP_PRO_GATED_MUL && (pro->unary < TLHIP_UNARY_NONE || pro->unary > TLHIP_UNARY_TANH))
    return set_error(TLHIP_ERR_INVALID, "%s: unknown unary op %d", who, pro->unary);
  if (pro->kind == TLHIP_PRO_RMSNORM && !(pro->eps >= 0.f))
    return set_error(TLHIP_ERR_INVALID, "%s: eps must be >= 0", who);
  if (p->m > 4)
    return set_error(TLHIP_ERR_UNSUPPORTED, "%s: the fused prologue is built for M <= 4, got %lld", who, (long long)p->m);
  p->pro.kind = pro->kind;
  p->pro.unary = pro->unary;
  p->pro.eps = pro->eps;
  p->pro.operand = pro->operand;
  return TLHIP_OK;
}

int tlhip_gemv_prologue(const tlhip_qweight_t* w, const tlhip_prologue_t* prologue, const void* x, int x_dtype,
                        int64_t m, void* y, int y_dtype, float alpha, const tlhip_epilogue_t* epilogue,
                        tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (!prologue || prologue->kind == TLHIP_PRO_NONE)
    return tlhip_gemv(w, x, x_dtype, m, y, y_dtype, alpha, epilogue, stream);
  Problem p;
  int rc = make_problem(w, x, x_dtype, m, y, y_dtype, alpha, epilogue, &p, "gemv_prologue");
  if (rc) return rc;
  rc = attach_prologue(prologue, &p, "gemv_prologue");
  if (rc) return rc;
  return launch_gemv(p, valu_config(p), resolve_stream(stream));
}

int tlhip_gemv_grouped_prologue(const tlhip_gemv_problem_t* problems, int count, const tlhip_prologue_t* prologue,
                                int x_dtype, int y_dtype, float alpha, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (!prologue || prologue->kind == TLHIP_PRO_NONE)
    return tlhip_gemv_grouped(problems, count, x_dtype, y_dtype, alpha, stream);
  if (count < 0 || (count > 0 && !problems))
    return set_error(TLHIP_ERR_INVALID, "gemv_grouped_prologue: bad problem list");
  if (count > 4)
    return set_error(TLHIP_ERR_INVALID, "gemv_grouped_prologue: a group holds at most 4 problems, got %d", count);
  Problem ps[4];
  for (int i = 0; i < count; ++i) {
    int rc = make_problem(&problems[i].w, problems[i].x, x_dtype, 1, problems[i].y, y_dtype, alpha,
                          problems[i].epilogue, &ps[i], "gemv_grouped_prologue");
    if (rc) return rc;
    rc = attach_prologue(prologue, &ps[i], "gemv_grouped_prologue");
    if (rc) return rc;
  }
  if (count == 0) return TLHIP_OK;
  hipStream_t s = resolve_stream(stream);
  int big = 0;
  for (int i = 1; i < count; ++i)
    if (ps[i].n > ps[big].n) big = i;
  const tlhip_kernel_config_t c = grouped_config(ps[big]);
  if (gemv_group_compatible(ps, count, c, nullptr)) return launch_gemv_grouped(ps, count, c, s);
  for (int i = 0; i < count; ++i) {
    int rc = launch_gemv(ps[i], valu_config(ps[i]), s);
    if (rc) return rc;
  }
  return TLHIP_OK;
}

int tlhip_gemm_prefill(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y, int y_dtype,
                       float alpha, const tlhip_epilogue_t* epilogue, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  Problem p;
  int rc = make_problem(w, x, x_dtype, m, y, y_dtype, alpha, epilogue, &p, "gemm_prefill");
  if (rc) return rc;
  if (x_dtype != TLHIP_F16) return set_error(TLHIP_ERR_INVALID, "gemm_prefill: activations must be f16");
  tlhip_kernel_config_t c = select_config(p);
  if (c.variant != VARIANT_TILED && c.variant != VARIANT_TILED_DIRECT) {
    c = tiled_cfg(p.m >= 128 ? 128 : 64, 128, 64, 2, 2);
    const char* why = nullptr;
    if (!gemm_config_applicable(p, c, &why))
      return set_error(TLHIP_ERR_INVALID, "gemm_prefill: shape not supported: %s", why ? why : "?");
  }
  return run_config(p, c, resolve_stream(stream));
}

int tlhip_matmul_quantized(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y,
                           int y_dtype, float alpha, const tlhip_epilogue_t* epilogue, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  Problem p;
  int rc = make_problem(w, x, x_dtype, m, y, y_dtype, alpha, epilogue, &p, "matmulQuantizedB");
  if (rc) return rc;
  if (p.m == 0 || p.n == 0) return TLHIP_OK;
  bool tune;
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    tune = (g_autotune_counter > 0 || env_autotune()) && !g_autotuning && g_tuned.count(problem_key(p)) == 0;
  }
  // f32 activations on the matrix-core route run the f16 problem's winner: nothing to tune here
  if (p.x_dtype == TLHIP_F32 && p.m >= kF32TiledFromRows) tune = false;
  if (tune) {
    // Lazy tuning at first dispatch (dispatch.ts:559-578), on the caller's stream; the
    // tuning launches write y, which the real launch below overwrites.  A problem whose
    // class already has a winner nearby gets the quick neighbour search.
    hipStream_t s = resolve_stream(stream);
    TuneOptions o;
    tlhip_kernel_config_t near;
    o.quick = class_config(p, &near);
    o.pool_bytes = (size_t)320 << 20;  // paid inside a caller's dispatch: just above the last-level cache
    // The tuning launches write y dozens of times.  A binary step whose input IS the output
    // (a residual added in place, a donated buffer) is correct in one launch, element by
    // element, and wrong from the second on: such a problem is tuned without its epilogue
    // (the key does not depend on the epilogue either).
    Problem tp = p;
    const char* y0 = (const char*)p.y;
    const char* y1 = y0 + (size_t)p.m * (size_t)p.n * (p.y_dtype == TLHIP_F16 ? 2 : 4);
    for (int i = 0; i < p.epi.n_ops; ++i) {
      if (p.epi.kind[i] != TLHIP_EPI_BINARY || !p.epi.input[i]) continue;
      const char* i0 = (const char*)p.epi.input[i];
      const char* i1 = i0 + (size_t)p.m * (size_t)p.n * (p.epi.input_dtype[i] == TLHIP_F16 ? 2 : 4);
      if (i0 < y1 && y0 < i1) tp.epi.n_ops = 0;
    }
    rc = autotune_problem(tp, {}, o, s, nullptr);
    if (rc) return rc;
  }
  return run_selected(p, select_config(p), resolve_stream(stream));
}

int tlhip_matmul_quantized_config(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y,
                                  int y_dtype, float alpha, const tlhip_epilogue_t* epilogue,
                                  const tlhip_kernel_config_t* config, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (!config) return set_error(TLHIP_ERR_INVALID, "matmul: null config");
  Problem p;
  int rc = make_problem(w, x, x_dtype, m, y, y_dtype, alpha, epilogue, &p, "matmulQuantizedB");
  if (rc) return rc;
  if (p.m == 0 || p.n == 0) return TLHIP_OK;
  const char* why = nullptr;
  if (!config_applicable(p, *config, &why))
    return set_error(TLHIP_ERR_INVALID, "matmul: config not applicable: %s", why ? why : "?");
  return matmul_with(p, *config, resolve_stream(stream));
}

static int shape_problem(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype, Problem* p) {
  int rc = validate_weight(w, "config");
  if (rc) return rc;
  memset(p, 0, sizeof *p);
  p->format = w->format;
  p->group_size = w->group_size;
  p->n = w->n;
  p->k = w->k;
  p->m = m;
  p->x_dtype = x_dtype;
  p->y_dtype = y_dtype;
  p->alpha = 1.f;
  return TLHIP_OK;
}

int tlhip_candidate_count(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype, int* out) {
  Problem p;
  int rc = shape_problem(w, x_dtype, m, y_dtype, &p);
  if (rc) return rc;
  if (!out) return set_error(TLHIP_ERR_INVALID, "candidate_count: null output");
  *out = (int)candidates(p).size();
  return TLHIP_OK;
}

int tlhip_candidate_get(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype, int index,
                        tlhip_kernel_config_t* out) {
  Problem p;
  int rc = shape_problem(w, x_dtype, m, y_dtype, &p);
  if (rc) return rc;
  auto c = candidates(p);
  if (!out || index < 0 || index >= (int)c.size())
    return set_error(TLHIP_ERR_INVALID, "candidate_get: index %d out of range [0,%d)", index, (int)c.size());
  *out = c[index];
  return TLHIP_OK;
}

int tlhip_selected_route(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype, int64_t* chunk_rows,
                         tlhip_kernel_config_t* first, tlhip_kernel_config_t* last) {
  Problem p;
  const int rc = shape_problem(w, x_dtype, m, y_dtype, &p);
  if (rc) return rc;
  if (!chunk_rows || !first || !last) return set_error(TLHIP_ERR_INVALID, "selected_route: null output");
  const Route r = plan_route(p, select_config(p));
  *chunk_rows = r.chunk;
  *first = r.first;
  *last = r.last;
  return TLHIP_OK;
}

int tlhip_selected_config(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype,
                          tlhip_kernel_config_t* out) {
  Problem p;
  int rc = shape_problem(w, x_dtype, m, y_dtype, &p);
  if (rc) return rc;
  if (!out) return set_error(TLHIP_ERR_INVALID, "selected_config: null output");
  *out = plan_route(p, select_config(p)).first;  // of the first launch, where the rows go in chunks
  if (p.x_dtype == TLHIP_F32 && p.m >= kF32TiledFromRows) {
    // what tlhip_matmul_quantized launches for these rows: the f16 problem's tiled kernel
    tlhip_kernel_config_t c = select_config(as_f16_activations(p));
    if (c.variant != VARIANT_TILED && c.variant != VARIANT_TILED_DIRECT) c = default_config(as_f16_activations(p));
    c.p5 = 0;  // as f32_rows_through_tiled launches it
    if (c.variant == VARIANT_TILED || c.variant == VARIANT_TILED_DIRECT) *out = c;
  }
  return TLHIP_OK;
}

int tlhip_tune_cache_seed(const tlhip_qweight_t* w, int x_dtype, int64_t m, int y_dtype,
                          const tlhip_kernel_config_t* config) {
  Problem p;
  int rc = shape_problem(w, x_dtype, m, y_dtype, &p);
  if (rc) return rc;
  if (!config) return set_error(TLHIP_ERR_INVALID, "tune_cache_seed: null config");
  const char* why = nullptr;
  if (!config_applicable(p, *config, &why))
    return set_error(TLHIP_ERR_INVALID, "tune_cache_seed: config not applicable: %s", why ? why : "?");
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  record_winner_locked(p, *config);
  return TLHIP_OK;
}

int tlhip_set_autotune_enabled(int enabled) {
  // dispatch.ts:128-134: true increments (nested regions), false resets to 0.
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  if (enabled) g_autotune_counter++;
  else g_autotune_counter = 0;
  return TLHIP_OK;
}

int tlhip_is_autotune_enabled(void) {
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  return g_autotune_counter > 0 || env_autotune();
}

int tlhip_autotune(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y, int y_dtype,
                   double* best_us) {
  return tlhip_autotune_pool(w, 1, x, x_dtype, m, y, y_dtype, nullptr, nullptr, nullptr, best_us);
}

int tlhip_autotune_pool(const tlhip_qweight_t* weights, int weight_count, const void* x, int x_dtype, int64_t m,
                        void* y, int y_dtype, const tlhip_epilogue_t* epilogue, const tlhip_autotune_options_t* options,
                        tlhip_stream_t stream, double* best_us) {
  TLHIP_REQUIRE_INIT();
  if (weight_count < 1 || !weights) return set_error(TLHIP_ERR_INVALID, "autotune: no weight");
  Problem p;
  int rc = make_problem(&weights[0], x, x_dtype, m, y, y_dtype, 1.f, epilogue, &p, "autotune");
  if (rc) return rc;
  if (p.m == 0 || p.n == 0 || p.k == 0) return set_error(TLHIP_ERR_INVALID, "autotune: empty problem");
  std::vector<WeightAlias> aliases;
  for (int i = 0; i < weight_count; ++i) {
    rc = validate_weight(&weights[i], "autotune");
    if (rc) return rc;
    if (weights[i].format != p.format || weights[i].n != p.n || weights[i].k != p.k ||
        (p.format != TLHIP_FMT_INT8_ROW && weights[i].group_size != p.group_size))
      return set_error(TLHIP_ERR_INVALID, "autotune: weight %d differs in format or shape from weight 0", i);
    aliases.push_back({weights[i].packed, weights[i].scales});
  }
  TuneOptions o;
  if (options) {
    if (options->reps > 0) o.reps = options->reps;
    if (options->batches > 0) o.batches = options->batches;
    if (options->retime_top > 0) o.retime_top = options->retime_top;
    if (options->warm_ms >= 0) o.warm_ms = options->warm_ms;
    o.quick = options->quick != 0;
    o.pool_bytes = (size_t)options->pool_bytes;
  }
  return autotune_problem(p, aliases, o, resolve_stream(stream), best_us);
}

int tlhip_pretune_matmul_shapes(const int64_t* mnk, int count) {
  if (count < 0 || (count > 0 && !mnk)) return set_error(TLHIP_ERR_INVALID, "pretune: bad arguments");
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  for (int i = 0; i < count; ++i) g_shape_hints.push_back({mnk[3 * i], mnk[3 * i + 1], mnk[3 * i + 2]});
  return TLHIP_OK;
}

int tlhip_tune_cache_export(char* buf, size_t cap, size_t* needed) {
  std::ostringstream os;
  os << "{\"version\":1,\"entries\":{";
  {
    std::lock_guard<std::mutex> lock(g_tune_mutex);
    bool first = true;
    for (auto& kv : g_tuned) {
      if (!first) os << ",";
      first = false;
      const auto& c = kv.second;
      os << "\"" << kv.first << "\":[" << c.variant << "," << c.p0 << "," << c.p1 << "," << c.p2 << "," << c.p3
         << "," << c.p4 << "," << c.p5 << "," << c.p6 << "]";
    }
  }
  os << "},\"model\":{";
  for (size_t i = 0; i < sizeof kModelFields / sizeof kModelFields[0]; ++i)
    os << (i ? "," : "") << "\"" << kModelFields[i].name << "\":" << g_model.*(kModelFields[i].field);
  os << "}}";
  const std::string s = os.str();
  if (needed) *needed = s.size() + 1;
  if (buf && cap > 0) {
    const size_t nc = std::min(cap - 1, s.size());
    memcpy(buf, s.data(), nc);
    buf[nc] = '\0';
  }
  return TLHIP_OK;
}

// Accepts exactly what export writes: {"version":1,"entries":{"key":[8 ints],...}}
int tlhip_tune_cache_import(const char* json) {
  if (!json) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: null text");
  const char* p = strstr(json, "\"entries\"");
  if (!p) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: no \"entries\" object");
  p = strchr(p, '{');
  if (!p) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: malformed entries");
  ++p;
  std::map<std::string, tlhip_kernel_config_t> parsed;
  for (;;) {
    while (*p == ' ' || *p == '\n' || *p == '\t' || *p == ',' || *p == '\r') ++p;
    if (*p == '}') break;
    if (*p != '"') return set_error(TLHIP_ERR_INVALID, "tune_cache_import: expected a key");
    const char* ke = strchr(p + 1, '"');
    if (!ke) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: unterminated key");
    std::string key(p + 1, ke);
    p = strchr(ke, '[');
    if (!p) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: expected an array for %s", key.c_str());
    ++p;
    int v[8];
    for (int i = 0; i < 8; ++i) {
      char* end = nullptr;
      v[i] = (int)strtol(p, &end, 10);
      if (end == p) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: expected 8 integers for %s", key.c_str());
      p = end;
      while (*p == ' ' || *p == ',' || *p == '\n' || *p == '\t' || *p == '\r') ++p;
    }
    if (*p != ']') return set_error(TLHIP_ERR_INVALID, "tune_cache_import: expected ] after %s", key.c_str());
    ++p;
    tlhip_kernel_config_t c = {v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]};
    parsed[key] = c;
  }
  // an optional "model" object: name : number pairs that override the routing model
  RouteModel model = g_model;
  if (const char* mp = strstr(json, "\"model\"")) {
    mp = strchr(mp, '{');
    if (!mp) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: malformed model");
    ++mp;
    for (;;) {
      while (*mp == ' ' || *mp == '\n' || *mp == '\t' || *mp == ',' || *mp == '\r') ++mp;
      if (*mp == '}') break;
      if (*mp != '"') return set_error(TLHIP_ERR_INVALID, "tune_cache_import: expected a model field name");
      const char* ke = strchr(mp + 1, '"');
      if (!ke) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: unterminated model field name");
      const std::string name(mp + 1, ke);
      mp = strchr(ke, ':');
      if (!mp) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: expected a value for model field %s", name.c_str());
      char* end = nullptr;
      const double v = strtod(mp + 1, &end);
      if (end == mp + 1 || !(v > 0.0) || v > 1e9)
        return set_error(TLHIP_ERR_INVALID, "tune_cache_import: model field %s needs a positive number", name.c_str());
      mp = end;
      bool known = false;
      for (const ModelField& f : kModelFields)
        if (name == f.name) model.*(f.field) = v, known = true;
      if (!known) return set_error(TLHIP_ERR_INVALID, "tune_cache_import: unknown model field %s", name.c_str());
    }
  }
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  g_model = model;
  for (auto& kv : parsed) {
    Problem q;
    if (parse_problem_key(kv.first, &q)) record_winner_locked(q, kv.second);  // the shape-class level too
    else g_tuned[kv.first] = kv.second;
  }
  return TLHIP_OK;
}

int tlhip_tune_cache_clear(void) {
  std::lock_guard<std::mutex> lock(g_tune_mutex);
  g_tuned.clear();
  g_class_tuned.clear();
  g_shape_hints.clear();
  g_model = RouteModel();
  return TLHIP_OK;
}

}  // extern "C"
