// Skinny GEMM (1 <= M <= 16) over int4 g32 weights on the matrix cores with the
// ACTIVATIONS HELD IN REGISTERS: no LDS staging of x, no barrier before the first
// weight is used, no LDS read per MFMA.
//
// gemv_mfma.hip stages the workgroup's K slice of x (M x K/ks f16) in LDS before
// anything else happens, and that copy is as many bytes per CU as the weights the
// CU streams (x: 32 bytes per k, weights: rows/2 bytes per k, 64 rows per CU at
// N = 4096): at M = 16 the kernel takes twice as long as at M = 1 although the
// weights are the same 25 MB.  Here all waves of a workgroup split the K slice of
// ONE 16-row block (wave w takes batches w, w + waves, ...: NSTEPS batches of U
// iterations of 128 k each) and walk over row blocks; a wave's part of x
// (16 rows x NSTEPS*U*128 k) is loaded once, straight from global memory in the
// MFMA's A-operand layout, into NSTEPS*U*16 registers, and stays there for every
// row block.
//
// Two schedules of the weight loads:
//  * ROUNDS = 0 (any number of row blocks per workgroup): the weights of the NEXT row
//    block (all NSTEPS*U 16-byte loads of a lane, plus their scales) are in flight
//    while the current one is consumed;
//  * ROUNDS = 1..4 (a workgroup has at most that many row blocks: the 9-28 MB decode
//    shapes on 256 CUs): EVERY weight load of the wave is issued before the first one
//    is consumed.  A 28 MB launch is three dependent round trips to HBM with the first
//    schedule and one with this; what a wave waits for afterwards is bandwidth.
//
// Several problems that share their activations (q/k/v, gate/up of a decode step)
// run as ONE launch: the row blocks of all problems form one index space, a row block
// finds its problem through a four-entry table.
//
// A = activations, B = weights, as in gemv_mfma.hip (same 4x4 word transpose, same
// exact integer f16 weights, scale applied to the f32 MFMA result).  The per-wave
// partial tiles of a row block are parked in LDS and combined once after the main
// loop behind one barrier; K slices across workgroups are combined by the last
// arriver in slice order, as in gemv_mfma.hip.
#include <cstring>

#include "gemv_mfma_common.h"

namespace tlhip {
namespace {

constexpr int kXMaxGroup = 4;

struct XregProblem {
  const u32x4* packed;
  const uint16_t* scales;
  void* y;
  int64_t n;
  int first_block;  // index of this problem's first 16-row block in the launch's block space
  DevEpilogue epi;
};

struct XregArgs {
  XregProblem p[kXMaxGroup];
  int count;
  const _Float16* x;
  float* workspace;
  int* counters;
  int k;
  int m;
  int nchunks;        // 16-byte chunks per weight row
  int groups_per_row;
  int ks;             // K slices handled by different workgroups (power of two)
  int ks_shift;
  int slice_iters;    // 128-k iterations per slice = waves * NSTEPS * U
  int nblocks;        // 16-row blocks of all problems together
  int xbar;           // 1: a workgroup barrier between the activation loads and the first weight load
  float alpha;
  int y_dtype;
};

template <int U, int NSTEPS, int MAXT, int ROUNDS>
__global__ __launch_bounds__(MAXT) void gemv_xreg_kernel(const XregArgs a) {
  extern __shared__ float parked[];  // [round][wave][256]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int waves = (int)(blockDim.x >> 6);
  const int nl = lane & 15;  // weight row in the block (B operand) / activation row (A operand)
  const int g = lane >> 4;   // k sub-block
  const int mrows = a.m;
  const int ml = nl < mrows ? nl : mrows - 1;  // rows beyond M alias the last row; never stored

  const int slice = blockIdx.x & (a.ks - 1);
  const int sets = gridDim.x >> a.ks_shift;
  const int rb0 = blockIdx.x >> a.ks_shift;
  const int rounds = (a.nblocks - rb0 + sets - 1) / sets;  // >= 1: sets <= nblocks
  const int it_begin = slice * a.slice_iters;

  // first iteration of this wave's batch s
  auto itb = [&](int s) { return it_begin + (wave + s * waves) * U; };

  // row block of the launch -> its problem (wave-uniform)
  auto problem_of = [&](int rb) {
    int pi = 0;
#pragma unroll
    for (int j = 1; j < kXMaxGroup; ++j)
      if (j < a.count && rb >= a.p[j].first_block) pi = j;
    return pi;
  };

  // ---- activations: unit (16 bytes = 8 k) 16*it + 4*t + g of row ml, for every MFMA
  // (s, u, t) of the wave, pair-permuted to the order the unpacked weights have.
  half8_t xa[NSTEPS][U][4];
  u32x4 raw[NSTEPS][U][4];
  {
    const u32x4* xrow = (const u32x4*)a.x + (size_t)ml * (a.k >> 3);
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s)
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < 4; ++t) raw[s][u][t] = xrow[(itb(s) + u) * 16 + 4 * t + g];
  }
  auto convert_x = [&]() {
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s)
#pragma unroll
      for (int u = 0; u < U; ++u)
#pragma unroll
        for (int t = 0; t < 4; ++t) xa[s][u][t] = __builtin_bit_cast(half8_t, permute_x_for_int4(raw[s][u][t]));
  };
  // The CU's memory pipeline takes requests in order: behind this barrier every wave's
  // activation loads (which come from L2) are queued ahead of every wave's weight
  // loads (which come from HBM).  The barrier waits for nothing but the waves' arrival.
  if (a.xbar) __builtin_amdgcn_s_barrier();

  // ---- the weights of one row block: raw loaded values only
  struct Round {
    u32x4 w[NSTEPS][U];
    uint32_t sv[NSTEPS][2 * U];  // scale 4u+t of batch s in half (t & 1) of word 2u + t/2
  };
  // In the hot loop a problem's fields are SELECTED from the four table entries, each read
  // with a constant index (scalar registers from the start of the kernel): a run-time index
  // into the kernel arguments would put scalar loads and their waits into every round.
  auto load_round = [&](Round& b, int r) {
    const int rb = min(rb0 + r * sets, a.nblocks - 1);  // a round past the end reloads the last block; never consumed
    const u32x4* packed = a.p[0].packed;
    const uint16_t* scales = a.p[0].scales;
    int64_t pn = a.p[0].n;
    int first = 0;
#pragma unroll
    for (int j = 1; j < kXMaxGroup; ++j) {
      const bool here = j < a.count && rb >= a.p[j].first_block;
      packed = here ? a.p[j].packed : packed;
      scales = here ? a.p[j].scales : scales;
      pn = here ? a.p[j].n : pn;
      first = here ? a.p[j].first_block : first;
    }
    const int64_t row = min((int64_t)(rb - first) * 16 + nl, pn - 1);  // tail rows reload the last row; never stored
    const u32x4* wrow = packed + row * a.nchunks;
    const uint16_t* srow = scales + row * a.groups_per_row;
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s) {
      const int it = itb(s);
#pragma unroll
      for (int u = 0; u < U; ++u) b.w[s][u] = __builtin_nontemporal_load(wrow + (it + u) * 4 + g);
      if (U == 1) {
        const uint2 v = *(const uint2*)(srow + it * 4);
        b.sv[s][0] = v.x;
        b.sv[s][1] = v.y;
      } else {
#pragma unroll
        for (int h = 0; h < U / 2; ++h) {
          const u32x4 v = *(const u32x4*)(srow + it * 4 + h * 8);  // 16-byte aligned: K % 256 == 0, it even
          b.sv[s][4 * h + 0] = v.x;
          b.sv[s][4 * h + 1] = v.y;
          b.sv[s][4 * h + 2] = v.z;
          b.sv[s][4 * h + 3] = v.w;
        }
      }
    }
  };

  auto compute_round = [&](const Round& b) {
    float4_t acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < NSTEPS; ++s)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        uint32_t w0 = b.w[s][u].x, w1 = b.w[s][u].y, w2 = b.w[s][u].z, w3 = b.w[s][u].w;
        transpose4(w0, w1, w2, w3);  // register t now holds word g of chunk 4*it+t
        const uint32_t ws[4] = {w0, w1, w2, w3};
        float4_t d[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          half2_t h[4];
          unpack_int4_word(ws[t], h);
          const float4_t zero = {0.f, 0.f, 0.f, 0.f};
          d[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[s][u][t], join8(h), zero, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t wd = b.sv[s][2 * u + (t >> 1)];
          const float sc = half_bits_to_float((t & 1) ? (wd >> 16) : (wd & 0xffffu));
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[q] = fmaf(sc, d[t][q], acc[q]);
        }
      }
    return acc;
  };

  auto park = [&](int r, const float4_t& acc) {
    float* tile = parked + (size_t)(r * waves + wave) * 256;
#pragma unroll
    for (int q = 0; q < 4; ++q) tile[(4 * g + q) * 16 + nl] = acc[q];
  };

  if constexpr (ROUNDS > 0) {
    // ---- every weight load of the wave first (rounds <= ROUNDS), then consume in order
    Round rd[ROUNDS];
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) load_round(rd[r], r);
    convert_x();
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      const float4_t acc = compute_round(rd[r]);
      if (r < rounds) park(r, acc);
    }
  } else {
    // ---- the next row block's loads are issued before the current one is consumed; two
    // register sets ping-pong, every load is unconditional (a round past the end reloads
    // the last row block and is not consumed).
    Round ra, rb_;
    load_round(ra, 0);
    convert_x();
    int r = 0;
    while (rounds - r >= 2) {
      load_round(rb_, r + 1);
      park(r, compute_round(ra));
      load_round(ra, r + 2);
      park(r + 1, compute_round(rb_));
      r += 2;
    }
    if (rounds - r == 1) park(r, compute_round(ra));
  }

  // ---- combine the waves' partial tiles, one row block per wave at a time
  lds_barrier();
  for (int t = wave; t < rounds; t += waves) {
    const int rb = rb0 + t * sets;
    const float* tiles = parked + (size_t)t * waves * 256;
    float4_t sum = {0.f, 0.f, 0.f, 0.f};
    for (int w = 0; w < waves; ++w) {
#pragma unroll
      for (int q = 0; q < 4; ++q) sum[q] += tiles[w * 256 + (4 * g + q) * 16 + nl];
    }
    bool owner = true;  // wave-uniform
    if (a.ks > 1) {
      // Publish this slice's tile; the workgroup that arrives last for the row block
      // adds the ks tiles in slice order (the sum does not depend on who is last),
      // resets the counter for the next launch and stores.  Device-scope relaxed
      // atomics only (coherent between the L2s by themselves); order: tile stores,
      // wait until they are acknowledged, then the counter.
      float* mine = a.workspace + ((size_t)rb * a.ks + slice) * 256;
#pragma unroll
      for (int q = 0; q < 4; ++q)
        __hip_atomic_store(mine + (4 * g + q) * 16 + nl, sum[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      int old = 0;
      if (lane == 0) old = __hip_atomic_fetch_add(a.counters + rb, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      old = __shfl(old, 0);
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
      owner = old == a.ks - 1;
      if (owner) {
        const float* all = a.workspace + (size_t)rb * a.ks * 256;
        sum = sum_slices(all, a.ks, (4 * g) * 16 + nl);
        if (lane == 0) __hip_atomic_store(a.counters + rb, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    if (owner) {
      const XregProblem& P = a.p[problem_of(rb)];
      const int64_t orow = (int64_t)(rb - P.first_block) * 16 + nl;
      if (orow < P.n) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int m = 4 * g + q;
          if (m < mrows) {
            const float v = apply_epilogue(P.epi, sum[q] * a.alpha, orow, (int64_t)m * P.n + orow);
            store_out(P.y, a.y_dtype, (int64_t)m * P.n + orow, v);
          }
        }
      }
    }
  }
}

struct XregGeometry {
  int grid, rounds, nsteps;
  size_t lds_bytes;
};

// waves, U, workgroups per CU, ks -> launch geometry for `nblocks` row blocks; false if
// the shape does not fit.  deep: every weight load upfront, at most 4 rounds.
bool xreg_geometry(int64_t k, int64_t nblocks, int waves, int unroll, int per_cu, int ks, bool deep, XregGeometry* out,
                   int* why) {
  const int64_t iters = k / 128;
  if (iters % ks != 0) return *why = 5, false;
  const int64_t slice_iters = iters / ks;
  if (slice_iters % ((int64_t)waves * unroll) != 0) return *why = 6, false;
  const int64_t nsteps = slice_iters / ((int64_t)waves * unroll);
  // registers: 28 per (step, iteration) for x and the two weight sets
  const int64_t nu = nsteps * unroll;
  if (nsteps < 1 || nu > (waves > 8 ? 2 : 6) || nsteps == 5) return *why = 6, false;
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  int64_t sets = (int64_t)cus * per_cu / ks;
  if (sets > nblocks) sets = nblocks;
  if (sets < 1) sets = 1;
  const int64_t rounds = (nblocks + sets - 1) / sets;
  if (deep) {
    // registers: 16 per iteration for x, 6 per (round, iteration) for the weights
    if (rounds > 4 || rounds * nu > 12) return *why = 9, false;
  }
  const size_t lds = (size_t)rounds * waves * 1024;
  if (lds * per_cu > 160 * 1024) return *why = 7, false;
  out->grid = (int)(sets * ks);
  out->rounds = (int)rounds;
  out->nsteps = (int)nsteps;
  out->lds_bytes = lds;
  return true;
}

template <int U, int NSTEPS, int ROUNDS>
const void* xreg_fn(int threads) {
  if (threads > 512) {
    if constexpr (U * NSTEPS <= 2) return (const void*)gemv_xreg_kernel<U, NSTEPS, 1024, ROUNDS>;
    else return nullptr;
  }
  return (const void*)gemv_xreg_kernel<U, NSTEPS, 512, ROUNDS>;
}

template <int U, int NSTEPS>
const void* xreg_fn_rounds(int threads, int rounds) {
  constexpr int NU = U * NSTEPS;
  switch (rounds) {
    case 0: return xreg_fn<U, NSTEPS, 0>(threads);
    case 1: return xreg_fn<U, NSTEPS, 1>(threads);
    case 2: return xreg_fn<U, NSTEPS, 2>(threads);
    case 3:
      if constexpr (NU * 3 <= 12) return xreg_fn<U, NSTEPS, 3>(threads);
      else return nullptr;
    case 4:
      if constexpr (NU * 4 <= 12) return xreg_fn<U, NSTEPS, 4>(threads);
      else return nullptr;
  }
  return nullptr;
}

// (iterations in flight, steps) -> kernel; rounds = 0: the ping-pong schedule.
const void* xreg_kernel_for(int unroll, int nsteps, int threads, int rounds) {
  switch (unroll * 10 + nsteps) {
    case 11: return xreg_fn_rounds<1, 1>(threads, rounds);
    case 12: return xreg_fn_rounds<1, 2>(threads, rounds);
    case 13: return xreg_fn_rounds<1, 3>(threads, rounds);
    case 14: return xreg_fn_rounds<1, 4>(threads, rounds);
    case 16: return xreg_fn_rounds<1, 6>(threads, rounds);
    case 21: return xreg_fn_rounds<2, 1>(threads, rounds);
    case 22: return xreg_fn_rounds<2, 2>(threads, rounds);
    case 23: return xreg_fn_rounds<2, 3>(threads, rounds);
    default: break;
  }
  return nullptr;
}

const char* const kXregReasons[] = {
    "not the gemv_mfma_xreg variant",
    "built for int4 weights with group size 32 and f16 activations",
    "M must be 1..16",
    "waves per workgroup must be 4, 8 or 16; iterations in flight 1 or 2; workgroups per CU 1, 2 or 4; p4 and p5 0 or 1",
    "K must be a multiple of 256",
    "K slices must be a power of two (1..16) that divides K/128",
    "the 128-k iterations of a K slice must be waves x steps x iterations in flight, with at most 6 (16 waves: 2) "
    "iterations per wave (their activations live in registers)",
    "one parked tile per round and wave does not fit LDS",
    "K slices need more partial-tile workspace or counters than the library holds",
    "every weight load upfront (p4 = 1): at most 4 row blocks per workgroup and 12 (row block, iteration) pairs per wave",
    "a group holds 1..4 problems that share activations, rows, format, group size, K and output type",
};

// The checks that depend on the problem class only (not on N).
int xreg_class_check(const Problem& p, const tlhip_kernel_config_t& c) {
  if (c.variant != VARIANT_GEMV_XREG) return 0;
  if (p.format != TLHIP_FMT_INT4_GROUPED || p.group_size != 32 || p.x_dtype != TLHIP_F16) return 1;
  if (p.m < 1 || p.m > 16) return 2;
  const int per_cu = c.p2 < 1 ? 1 : c.p2;
  if ((c.p0 != 4 && c.p0 != 8 && c.p0 != 16) || (c.p1 != 1 && c.p1 != 2) || (per_cu != 1 && per_cu != 2 && per_cu != 4) ||
      (c.p4 != 0 && c.p4 != 1) || (c.p5 != 0 && c.p5 != 1))
    return 3;
  if (p.k % 256 != 0 || p.k <= 0) return 4;
  const int ks = c.p3 < 1 ? 1 : c.p3;
  if (ks > 16 || (ks & (ks - 1)) != 0) return 5;
  return -1;
}

}  // namespace

bool gemv_xreg_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why) {
  auto fail = [&](int i) {
    if (why) *why = kXregReasons[i];
    return false;
  };
  const int cls = xreg_class_check(p, c);
  if (cls >= 0) return fail(cls);
  const int per_cu = c.p2 < 1 ? 1 : c.p2, ks = c.p3 < 1 ? 1 : c.p3;
  const int64_t nblocks = (p.n + 15) / 16;
  XregGeometry geo;
  int w = 0;
  if (!xreg_geometry(p.k, nblocks, c.p0, c.p1, per_cu, ks, c.p4 == 1, &geo, &w)) return fail(w);
  if (!xreg_kernel_for(c.p1, geo.nsteps, c.p0 * 64, c.p4 == 1 ? geo.rounds : 0)) return fail(c.p4 == 1 ? 9 : 6);
  if (ks > 1 && (nblocks > scratch_counters(p) || (size_t)nblocks * ks * 256 > scratch_tile_floats(p))) return fail(8);
  return true;
}

// The problems of a group: same activations and rows, one shape class; N, pointers and
// epilogues per problem.  The configuration is checked against the group's total rows.
bool gemv_xreg_group_applicable(const Problem* ps, int count, const tlhip_kernel_config_t& c, const char** why) {
  auto fail = [&](int i) {
    if (why) *why = kXregReasons[i];
    return false;
  };
  if (count < 1 || count > kXMaxGroup) return fail(10);
  int64_t nblocks = 0;
  for (int i = 0; i < count; ++i) {
    if (ps[i].x != ps[0].x || ps[i].m != ps[0].m || ps[i].format != ps[0].format || ps[i].group_size != ps[0].group_size ||
        ps[i].k != ps[0].k || ps[i].x_dtype != ps[0].x_dtype || ps[i].y_dtype != ps[0].y_dtype || ps[i].alpha != ps[0].alpha)
      return fail(10);
    nblocks += (ps[i].n + 15) / 16;
  }
  const int cls = xreg_class_check(ps[0], c);
  if (cls >= 0) return fail(cls);
  if (nblocks == 0) return true;
  const int per_cu = c.p2 < 1 ? 1 : c.p2, ks = c.p3 < 1 ? 1 : c.p3;
  XregGeometry geo;
  int w = 0;
  if (!xreg_geometry(ps[0].k, nblocks, c.p0, c.p1, per_cu, ks, c.p4 == 1, &geo, &w)) return fail(w);
  if (!xreg_kernel_for(c.p1, geo.nsteps, c.p0 * 64, c.p4 == 1 ? geo.rounds : 0)) return fail(c.p4 == 1 ? 9 : 6);
  if (ks > 1 && (nblocks > scratch_counters(ps[0]) || (size_t)nblocks * ks * 256 > scratch_tile_floats(ps[0]))) return fail(8);
  return true;
}

int launch_gemv_xreg_group(const Problem* ps, int count, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_xreg_group_applicable(ps, count, c, &why))
    return set_error(TLHIP_ERR_INVALID, "gemv_mfma_xreg: config not applicable: %s", why);
  const int waves = c.p0, unroll = c.p1, per_cu = c.p2 < 1 ? 1 : c.p2, ks = c.p3 < 1 ? 1 : c.p3;
  XregArgs a;
  memset(&a, 0, sizeof a);
  int64_t nblocks = 0;
  for (int i = 0; i < count; ++i) {
    if (ps[i].n == 0) continue;
    XregProblem& P = a.p[a.count++];
    P.packed = (const u32x4*)ps[i].packed;
    P.scales = (const uint16_t*)ps[i].scales;
    P.y = ps[i].y;
    P.n = ps[i].n;
    P.first_block = (int)nblocks;
    P.epi = ps[i].epi;
    nblocks += (ps[i].n + 15) / 16;
  }
  if (a.count == 0 || ps[0].m == 0) return TLHIP_OK;
  const Problem& p = ps[0];
  XregGeometry geo;
  int w = 0;
  if (!xreg_geometry(p.k, nblocks, waves, unroll, per_cu, ks, c.p4 == 1, &geo, &w))
    return set_error(TLHIP_ERR_INVALID, "gemv_mfma_xreg: launch geometry does not close");
  a.x = (const _Float16*)p.x;
  a.workspace = nullptr;
  a.counters = nullptr;
  if (ks > 1) {
    const int rc = problem_scratch(p, stream, &a.workspace, &a.counters);
    if (rc) return rc;
  }
  a.k = (int)p.k;
  a.m = (int)p.m;
  a.nchunks = (int)(p.k / 32);
  a.groups_per_row = (int)(p.k / 32);
  a.ks = ks;
  a.ks_shift = __builtin_ctz((unsigned)ks);
  a.slice_iters = (int)(p.k / 128 / ks);
  a.nblocks = (int)nblocks;
  a.xbar = c.p5;
  a.alpha = p.alpha;
  a.y_dtype = p.y_dtype;
  const int threads = waves * 64;
  const void* fn = xreg_kernel_for(unroll, geo.nsteps, threads, c.p4 == 1 ? geo.rounds : 0);
  if (!fn) return set_error(TLHIP_ERR_INVALID, "gemv_mfma_xreg: no kernel instance for this configuration");
  void* args[] = {(void*)&a};
  const int rc = launch_kernel(fn, dim3(geo.grid), dim3(threads), args, geo.lds_bytes, stream);
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  for (int i = 0; i < a.count; ++i) count_gemv_dispatch();
  return TLHIP_OK;
}

int launch_gemv_xreg(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream) {
  const char* why = nullptr;
  if (!gemv_xreg_config_applicable(p, c, &why))
    return set_error(TLHIP_ERR_INVALID, "gemv_mfma_xreg: config not applicable: %s", why);
  if (p.n == 0 || p.m == 0) return TLHIP_OK;
  return launch_gemv_xreg_group(&p, 1, c, stream);
}

// Every instance launch_gemv_xreg can reach, in prepare mode (see launch_kernel).
int prepare_gemv_xreg_kernels() {
  static const int un[][2] = {{1, 1}, {1, 2}, {1, 3}, {1, 4}, {1, 6}, {2, 1}, {2, 2}, {2, 3}};
  for (auto& c : un)
    for (int threads : {512, 1024})
      for (int rounds = 0; rounds <= 4; ++rounds) {
        const void* fn = xreg_kernel_for(c[0], c[1], threads, rounds);
        if (!fn) continue;
        const int rc = launch_kernel(fn, dim3(1), dim3(64), nullptr, 0, nullptr);
        if (rc) return rc;
      }
  return TLHIP_OK;
}

}  // namespace tlhip
