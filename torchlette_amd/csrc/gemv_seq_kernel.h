// A SEQUENCE of skinny GEMMs (decode Linears, 1 <= M <= 16 rows, int4 weights in groups
// of 32, f16 activations) in ONE launch: the weight stream of the next Linear starts while
// the previous one is still being finished, and a Linear that reads what an earlier one of
// the launch wrote (down after gate/up in an MLP block) is ordered behind it inside the
// kernel instead of behind a kernel boundary.
//
// Units.  The row blocks (16 weight rows) of every problem are cut into units of 4: a unit
// is "4 row blocks of one problem over all of K", and the units of all problems, in problem
// order, form one sequence that is dealt round-robin to the workgroups (unit u goes to
// workgroup u mod grid, which works through its units in order).  A GATED problem
// (y = act(x Wg^T) * (x Wu^T), the MLP's gate and up projections) puts 2 row blocks of Wg
// and the same 2 of Wu into a unit, so that act(gate) * up is formed in registers and only
// the product is written.
// Inside a unit the work is that of gemv_wave_kernel.h: the workgroup's waves split K into
// W contiguous ranges of `steps` 128-k steps; for a step a wave loads its 128 k of the
// activations (whole rows, coalesced, through a wave-private LDS patch into the MFMA A
// operand layout) and the 16 x 64 bytes of packed weights of each of the unit's 4 row
// blocks, D steps ahead of the one it computes; the scales of the wave's whole K range are
// loaded once per unit as 16-byte pieces laid side by side in the wave's LDS.  The ring of D
// register sets runs ACROSS unit and problem boundaries: the loads of a wave's next unit
// are in flight while the current unit is finished (partial tiles parked in LDS, one
// barrier, all threads add the W partials in wave order, epilogue, store; parked tiles
// double buffered).
//
// Order between problems.  `done` (device memory) counts finished units.  A problem marked
// `wait` starts only when every unit in front of its first one is done: the workgroup lets
// its ring drain, wave 0 polls `done` (bounded: after `spin_limit` polls it sets `error`,
// and the workgroup leaves), everybody meets at a barrier, acquires at agent scope, and the
// ring is primed again.  A unit of a problem that somebody waits for (`signal`) is counted
// only after every thread of the workgroup has released its stores at agent scope.  Unit u
// only ever waits for units with smaller numbers, and every workgroup takes its units in
// increasing order, so with all workgroups resident (the host checks) nobody waits in a
// cycle.  The last workgroup to leave clears the counters for the next launch.
//
// Every load of the steady state is unconditional and goes to a valid address (see
// gemv_wave_kernel.h): a ring slot with nothing to load (past the last unit, or in front
// of a wait) takes the same instructions at offset 0.
#pragma once
#include <cstddef>
#include <cstring>

#include "gemv_mfma_common.h"

namespace tlhip {

constexpr int kSeqMaxProblems = 16;
constexpr int kSeqSlots = 4;        // row-block slots of a unit
constexpr int kSeqScaleLoads = 6;   // 16-byte scale loads per lane and unit at most

struct SeqProblem {
  const void* packed[2];   // [1]: the up matrix of a gated pair, else the same as [0]
  const void* scales[2];
  const void* x;
  void* y;
  uint32_t packed_bytes, scales_bytes, x_bytes;
  int n;
  int kb;          // bytes of a packed weight row, K / 2
  int nsteps;      // 128-k steps over all of K
  int steps;       // steps per wave: ceil(nsteps / waves)
  int spr;         // 16-byte scale pieces per row of a wave's (16-byte aligned) window
  int spr_recip;   // ceil(65536 / spr)
  int first_unit;  // the problem's first unit in the launch's sequence
  int gated;       // 1: a unit holds 2 row blocks of packed[0] and the same 2 of packed[1]
  int wait;        // 1: starts only when all units in front of first_unit are done
  int signal;      // 1: a later problem waits for this one's output
  int y_dtype;
  float alpha;
  DevEpilogue epi;
};

// Device state of sequence launches on one stream: zero between launches, except `error`,
// which stays set once a wait has expired.
struct SeqState {
  uint32_t done;    // units finished
  uint32_t exited;  // workgroups that have left; the last one clears both counters
  uint32_t error;
  uint32_t pad;
};

struct SeqTable {
  int count;
  int m;
  int total_units;
  int fault;  // test hook: added to every wait's threshold, so that no wait can be satisfied
  uint32_t spin_limit;  // polls a wait may take
  SeqState* state;
  SeqProblem p[kSeqMaxProblems];
};

namespace {

__device__ __forceinline__ __amdgpu_buffer_rsrc_t seq_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, (int)bytes, 0x00020000);
}

// MQ: 16-byte activation loads per lane and step (they cover 4 MQ rows >= M); D: steps in flight.
template <int MQ, int D>
__global__ __launch_bounds__(512) void gemv_seq_kernel(const SeqTable a) {
  constexpr int RP = kSeqSlots;
  constexpr int RU = 17;  // units of a patch row: 128 k of f16 + 1 pad
  constexpr int WAVE_UNITS = 16 * RU + kSeqScaleLoads * 64;
  extern __shared__ u32x4 lds[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int W = (int)(blockDim.x >> 6);
  const int nl = lane & 15;  // weight row inside a block (B operand), activation row (A operand)
  const int g = lane >> 4;   // k sub-block
  const int wg = blockIdx.x, nwg = gridDim.x;
  u32x4* patch = lds + wave * WAVE_UNITS;
  u32x4* sarea = patch + 16 * RU;                      // [slot][row][spr pieces]
  float* parked = (float*)(lds + W * WAVE_UNITS);      // [2][wave][RP][256]
  int* flag = (int*)(parked + 2 * W * RP * 256);
  const int mrows = a.m;

  // A cursor: the unit it is in (the i-th of this workgroup) and its step.
  struct Cur {
    int i, j;
    bool live;  // false: past the workgroup's last unit
    int pi;     // problem of the unit
    __amdgpu_buffer_rsrc_t bw0, bw1, bs0, bs1, bx;
    int n, kb, nsteps, steps, spr, spr_recip, rb0, gated, wait, first_unit, row_sbytes;
  };
  auto enter = [&](Cur& c, int i) __attribute__((always_inline)) {
    const int u = wg + i * nwg;
    c.i = i;
    c.j = 0;
    c.live = u < a.total_units;
    if (c.live) {
      int pi = 0;
#pragma unroll
      for (int q = 1; q < kSeqMaxProblems; ++q)
        if (q < a.count && u >= a.p[q].first_unit) pi = q;
      const SeqProblem& P = a.p[pi];
      c.pi = pi;
      c.bw0 = seq_rsrc(P.packed[0], P.packed_bytes);
      c.bw1 = seq_rsrc(P.packed[1], P.packed_bytes);
      c.bs0 = seq_rsrc(P.scales[0], P.scales_bytes);
      c.bs1 = seq_rsrc(P.scales[1], P.scales_bytes);
      c.bx = seq_rsrc(P.x, P.x_bytes);
      c.n = P.n;
      c.kb = P.kb;
      c.nsteps = P.nsteps;
      c.steps = P.steps;
      c.spr = P.spr;
      c.spr_recip = P.spr_recip;
      c.gated = P.gated;
      c.wait = P.wait;
      c.first_unit = P.first_unit;
      c.rb0 = (u - P.first_unit) * (P.gated ? 2 : 4);
      c.row_sbytes = P.kb >> 3;  // bytes of a row's scales, K / 16
    }
  };

  u32x4 rw[D][RP];
  u32x4 rx[D][MQ];
  u32x4 sreg[kSeqScaleLoads];
  bool live[D];

  const int xrow0 = lane >> 4;
  const int xunit = lane & 15;

  // The loads of the step at `c` into ring slot s, or (on = false) the same instructions at
  // offset 0.  With the unit's first step: the scales of the wave's K range.
  auto issue = [&](int s, const Cur& c, bool on) __attribute__((always_inline)) {
    const int st0 = wave * c.steps;
    const int st = st0 + c.j;
    const int mask = -(int)(on & (st < c.nsteps));
#pragma unroll
    for (int q = 0; q < MQ; ++q) {
      const int row = min(4 * q + xrow0, mrows - 1);
      rx[s][q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(c.bx, (row * (c.kb * 4) + st * 256 + xunit * 16) & mask, 0, 0));
    }
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      const int row = (c.rb0 + (r >> c.gated)) * 16 + nl;
      const int off = (row * c.kb + st * 64 + g * 16) & mask & -(int)(row < c.n);
      rw[s][r] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128((r & 1) ? c.bw1 : c.bw0, off, 0, 2));
    }
    if (on && c.j == 0) {
      // window: from the 16-byte boundary at or below the wave's first scale; group h of
      // the loads takes the slots h and h + 2 (one matrix per instruction)
      const int wstart = (st0 * 8) & ~15;
#pragma unroll
      for (int i = 0; i < kSeqScaleLoads; ++i) {
        const int h = i / (kSeqScaleLoads / 2);
        const int f = (i % (kSeqScaleLoads / 2)) * 64 + lane;
        const int ri = (f * c.spr_recip) >> 16;  // f / spr (exact for f < 192, spr <= 24)
        const int piece = f - ri * c.spr;
        const int slot = h + 2 * (ri >> 4);
        const int row = (c.rb0 + (slot >> c.gated)) * 16 + (ri & 15);
        const int pofs = wstart + piece * 16;
        const int ok = (int)(ri < 32) & (int)(row < c.n) & (int)(pofs < c.row_sbytes);
        sreg[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(h ? c.bs1 : c.bs0, (row * c.row_sbytes + pofs) & -ok, 0, 0));
      }
    }
  };

  float4_t acc[RP];
#pragma unroll
  for (int r = 0; r < RP; ++r) acc[r] = (float4_t){0.f, 0.f, 0.f, 0.f};
  int finished = 0;  // units this workgroup has finished: the parity of the parked tiles

  // End of a unit: park, one barrier, all threads combine and store; then the unit is counted.
  auto finish = [&](const Cur& c) __attribute__((always_inline)) {
    float* buf = parked + (finished & 1) * (W * RP * 256);
    ++finished;
#pragma unroll
    for (int r = 0; r < RP; ++r) {
#pragma unroll
      for (int q = 0; q < 4; ++q) buf[(wave * RP + r) * 256 + (4 * g + q) * 16 + nl] = acc[r][q];
      acc[r] = (float4_t){0.f, 0.f, 0.f, 0.f};
    }
    lds_barrier();
    const SeqProblem& P = a.p[c.pi];
    const int gated = P.gated;
    const int outs = gated ? 2 * 256 : 4 * 256;
    for (int o = tid; o < outs; o += (int)blockDim.x) {
      const int b = o >> 8, e = o & 255;  // row block of the unit, element of its tile
      const int r0 = gated ? 2 * b : b;
      float s0 = 0.f, s1 = 0.f;
      for (int w = 0; w < W; ++w) {
        s0 += buf[(w * RP + r0) * 256 + e];
        if (gated) s1 += buf[(w * RP + r0 + 1) * 256 + e];
      }
      const int m = e >> 4;
      const int col = (c.rb0 + b) * 16 + (e & 15);
      if (col < P.n && m < mrows) {
        const int64_t idx = (int64_t)m * P.n + col;
        float v = apply_epilogue(P.epi, s0 * P.alpha, col, idx);
        if (gated) v *= s1 * P.alpha;
        store_out(P.y, P.y_dtype, idx, v);
      }
    }
    if (P.signal) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "agent");
      __builtin_amdgcn_s_barrier();
    }
    if (tid == 0) __hip_atomic_fetch_add(&a.state->done, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  auto consume = [&](int s, const Cur& c) __attribute__((always_inline)) {
    const int st0 = wave * c.steps;
    if (c.j == 0) {
      // the unit's scales (issued with its first step): into the wave's LDS
#pragma unroll
      for (int i = 0; i < kSeqScaleLoads; ++i) {
        const int h = i / (kSeqScaleLoads / 2);
        const int f = (i % (kSeqScaleLoads / 2)) * 64 + lane;
        const int ri = (f * c.spr_recip) >> 16;
        const int piece = f - ri * c.spr;
        const int slot = h + 2 * (ri >> 4);
        if (ri < 32) sarea[(slot * 16 + (ri & 15)) * c.spr + piece] = sreg[i];
      }
    }
    if (st0 + c.j < c.nsteps) {  // wave-uniform: a step beyond K adds nothing
#pragma unroll
      for (int q = 0; q < MQ; ++q) patch[(4 * q + xrow0) * RU + xunit] = permute_x_for_int4(rx[s][q]);
      half8_t xa[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) xa[t] = __builtin_bit_cast(half8_t, patch[nl * RU + 4 * t + g]);
      const int sbyte = ((st0 * 8) & 15) + c.j * 8;  // this step's scales inside the window
#pragma unroll
      for (int r = 0; r < RP; ++r) {
        const uint2 sv = *(const uint2*)((const char*)(sarea + (r * 16 + nl) * c.spr) + sbyte);
        uint32_t w0 = rw[s][r].x, w1 = rw[s][r].y, w2 = rw[s][r].z, w3 = rw[s][r].w;
        transpose4(w0, w1, w2, w3);  // register t now holds word g of chunk 4*it + t
        const uint32_t ws[4] = {w0, w1, w2, w3};
        float4_t d[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          half2_t h[4];
          unpack_int4_word(ws[t], h);
          const float4_t zero = {0.f, 0.f, 0.f, 0.f};
          d[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(xa[t], join8(h), zero, 0, 0, 0);
        }
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t wd = (t >> 1) ? sv.y : sv.x;
          const float sc = half_bits_to_float((t & 1) ? (wd >> 16) : (wd & 0xffffu));
#pragma unroll
          for (int q = 0; q < 4; ++q) acc[r][q] = fmaf(sc, d[t][q], acc[r][q]);
        }
      }
    }
    if (c.j == c.steps - 1) finish(c);
  };

  Cur ci, cc;
  enter(ci, 0);
  if (ci.live) {
    cc = ci;
    uint32_t waited = 0;  // units known to be done (the largest threshold waited for)
    // the issue cursor stands in front of a unit that has to wait
    bool blocked = ci.wait && (uint32_t)(ci.first_unit + a.fault) > waited;
    bool abort = false;
    auto advance_issue = [&]() __attribute__((always_inline)) {
      if (++ci.j == ci.steps) {
        enter(ci, ci.i + 1);
        blocked = ci.live && ci.wait && (uint32_t)(ci.first_unit + a.fault) > waited;
      }
    };
#pragma unroll
    for (int s = 0; s < D; ++s) {
      const bool on = ci.live && !blocked;
      issue(s, ci, on);
      live[s] = on;
      if (on) advance_issue();
    }
    while (cc.live) {
      bool any = false;
#pragma unroll
      for (int s = 0; s < D; ++s) any |= live[s];
      if (!any) {
        // the ring is empty: the issue cursor waits for the units in front of its problem
        // (cc.live and an empty ring: nothing else stops the issue cursor)
        const uint32_t need = (uint32_t)(ci.first_unit + a.fault);
        if (wave == 0) {
          uint32_t seen = 0;
          const uint32_t limit = a.spin_limit;
          for (uint32_t spin = 0; spin < limit; ++spin) {
            seen = __hip_atomic_load(&a.state->done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (seen >= need) break;
            __builtin_amdgcn_s_sleep(2);
          }
          if (lane == 0) {
            *flag = seen >= need ? 1 : 0;
            if (seen < need) __hip_atomic_fetch_or(&a.state->error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        lds_barrier();
        abort = *flag == 0;
        lds_barrier();  // nobody rewrites the flag before everybody has read it
        if (abort) break;
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
        waited = need;
        blocked = false;
      }
#pragma unroll
      for (int s = 0; s < D; ++s) {
        if (live[s]) {
          consume(s, cc);
          if (++cc.j == cc.steps) enter(cc, cc.i + 1);
        }
        const bool on = ci.live && !blocked;
        issue(s, ci, on);
        live[s] = on;
        if (on) advance_issue();
      }
    }
  }
  // ---- leave: the last workgroup clears the counters for the next launch
  __builtin_amdgcn_s_barrier();
  if (tid == 0) {
    const uint32_t old = __hip_atomic_fetch_add(&a.state->exited, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
    if (old == (uint32_t)nwg - 1) {
      __hip_atomic_store(&a.state->done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(&a.state->exited, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
}

}  // namespace
}  // namespace tlhip
