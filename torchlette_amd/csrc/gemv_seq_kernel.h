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
// cycle.  The counters only grow; the host tells a launch where they stood before it.
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
  int nrb;         // row-block slots a unit uses, 1..4 (gated: 2 or 4, a pair of slots per row block)
  int gated;       // 1: a unit holds row blocks of packed[0] and the same ones of packed[1], side by side
  int wait;        // 1: starts only when all units in front of first_unit are done
  int signal;      // 1: a later problem waits for this one's output
  int y_dtype;
  float alpha;
  DevEpilogue epi;
};

// Device state of sequence launches on one stream.  Finished units are counted in 16 shards
// on cache lines of their own (one counter for the whole chip made every workgroup's
// increment queue behind 255 others: 20 us per launch); a workgroup adds to shard
// (workgroup mod 16), a waiting workgroup adds the shards up.  The counters only grow: the
// host hands every launch the sum they held before it (`base`), so nothing is cleared
// between launches.  `error` stays set once a wait has expired.
constexpr int kSeqShards = 16;
struct SeqState {
  uint32_t done[kSeqShards][16];  // [shard][0] counts; the rest pads the shard to 64 bytes
  uint32_t error;
  uint32_t pad[15];
};

constexpr int kAuxAgentScope = 16;  // the sc1 bit of a buffer load's cache policy on gfx942 / gfx950

struct SeqTable {
  int count;
  int m;
  int total_units;
  int fault;  // test hook: added to every wait's threshold, so that no wait can be satisfied
  int counting;  // 1: some problem waits, so finished units are counted (0: no counter is touched)
  uint32_t base;  // what the shards of `done` add up to when the launch starts
  uint32_t spin_limit;  // polls a wait may take
  SeqState* state;
  SeqProblem p[kSeqMaxProblems];
};

namespace {

// Pointers into device memory, said to be so: through a generic pointer the compiler emits
// FLAT instructions, which may complete out of order with the buffer loads, and from the
// first one on every wait for a load becomes a wait for all of them.
#define TLHIP_GLOBAL __attribute__((address_space(1)))
template <typename T>
__device__ __forceinline__ T TLHIP_GLOBAL* as_global(const void* p) {
  return (T TLHIP_GLOBAL*)(uintptr_t)p;
}

// A wave-uniform word of the problem table's copy in LDS, as a scalar.
__device__ __forceinline__ int lds_word(const void* p) { return __builtin_amdgcn_readfirstlane(*(const int*)p); }
__device__ __forceinline__ const void* lds_pointer(const void* p) {
  const uint64_t lo = (uint32_t)lds_word(p), hi = (uint32_t)lds_word((const char*)p + 4);
  return (const void*)(lo | (hi << 32));
}

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
  // The problem table: one cooperative copy from the kernel arguments into LDS, read from
  // there afterwards.  (The argument block may live in host memory: a scalar load from it
  // that misses is a trip over the bus, and walking sixteen 200-byte entries that way
  // cost a launch 10 us.)
  const SeqProblem* table = (const SeqProblem*)(flag + 4);
  {
    typedef const u32x4 __attribute__((address_space(4))) * KernargUnits;
    KernargUnits src = (KernargUnits)((const char __attribute__((address_space(4)))*)__builtin_amdgcn_kernarg_segment_ptr() +
                                      offsetof(SeqTable, p));
    u32x4* dst = (u32x4*)table;
    const int units = a.count * (int)(sizeof(SeqProblem) / 16);
    for (int i = tid; i < units; i += (int)blockDim.x) dst[i] = src[i];
    lds_barrier();
  }

  // A unit of this workgroup (its i-th) with the fields of its problem, as scalars.
  struct Unit {
    __amdgpu_buffer_rsrc_t bw0, bw1, bs0, bs1, bx;
    int i;
    int live;  // 0: past the workgroup's last unit
    int pi;    // problem of the unit
    int n, kb, nsteps, steps, steps_p, spr, spr_recip, rb0, nrb, gated, wait, first_unit, row_sbytes;
  };
  static_assert(sizeof(Unit) == 5 * 16 + 16 * 4, "no padding: a copy of a unit is register moves");
  auto enter = [&](Unit& c, int i) __attribute__((always_inline)) {
    const int u = wg + i * nwg;
    c.i = i;
    c.live = (int)(u < a.total_units);
    if (c.live) {
      int pi = 0;
      for (int q = 1; q < a.count; ++q)
        if (u >= lds_word(&table[q].first_unit)) pi = q;
      const SeqProblem& P = table[pi];
      c.pi = pi;
      const uint32_t packed_bytes = (uint32_t)lds_word(&P.packed_bytes), scales_bytes = (uint32_t)lds_word(&P.scales_bytes);
      c.bw0 = seq_rsrc(lds_pointer(&P.packed[0]), packed_bytes);
      c.bw1 = seq_rsrc(lds_pointer(&P.packed[1]), packed_bytes);
      c.bs0 = seq_rsrc(lds_pointer(&P.scales[0]), scales_bytes);
      c.bs1 = seq_rsrc(lds_pointer(&P.scales[1]), scales_bytes);
      c.bx = seq_rsrc(lds_pointer(&P.x), (uint32_t)lds_word(&P.x_bytes));
      c.n = lds_word(&P.n);
      c.kb = lds_word(&P.kb);
      c.nsteps = lds_word(&P.nsteps);
      c.steps = lds_word(&P.steps);
      c.steps_p = (c.steps + D - 1) / D * D;
      c.spr = lds_word(&P.spr);
      c.spr_recip = lds_word(&P.spr_recip);
      c.nrb = lds_word(&P.nrb);
      c.gated = lds_word(&P.gated);
      c.wait = lds_word(&P.wait);
      c.first_unit = lds_word(&P.first_unit);
      c.rb0 = (u - c.first_unit) * (c.nrb >> c.gated);
      c.row_sbytes = c.kb >> 3;  // bytes of a row's scales, K / 16
    }
  };

  u32x4 rw[D][RP];
  u32x4 rx[D][MQ];
  u32x4 sreg[kSeqScaleLoads];

  const int xrow0 = lane >> 4;
  const int xunit = lane & 15;

  // The loads of step j of unit `c` into ring slot s, or (on = false, a step beyond the
  // wave's K range, a row-block slot the unit does not use) the same instructions at offset 0.
  auto issue = [&](int s, const Unit& c, int j, bool on) __attribute__((always_inline)) {
    const int st = wave * c.steps + j;
    const bool step_on = on & (j < c.steps) & (st < c.nsteps);  // wave-uniform
    const int mask = -(int)step_on;
#pragma unroll
    for (int q = 0; q < MQ; ++q) {
      const int row = min(4 * q + xrow0, mrows - 1);
      // The activations of a step that waits were written by other workgroups of this
      // launch, so they are loaded at agent scope (sc1: never served from a stale line of
      // this XCD's L2 or of the vector cache); those of other steps too, because a second
      // form of the load under a condition multiplies the paths through the unit loop.
      rx[s][q] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(c.bx, (row * (c.kb * 4) + st * 256 + xunit * 16) & mask, 0, kAuxAgentScope));
    }
#pragma unroll
    for (int r = 0; r < RP; ++r) {
      // A slot with nothing to load reads a line of the activations instead (this wave's own
      // 64 bytes of the first 512, which its CU has just had in hand): the same
      // instruction, but no trip to memory.  (At offset 0 of the weights, where every wave
      // of the chip then reads one line with the streaming hint, such loads cost a launch
      // tens of microseconds.)
      const bool use = step_on & (r < c.nrb);  // wave-uniform
      const int row = (c.rb0 + (r >> c.gated)) * 16 + nl;
      const int off = use ? ((row * c.kb + st * 64 + g * 16) & -(int)(row < c.n)) : (wave & 7) * 64;
      rw[s][r] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(use ? ((r & 1) ? c.bw1 : c.bw0) : c.bx, off, 0, 2));
    }
  };
  // The scales of the wave's K range of unit `c`.  Window: from the 16-byte boundary at or
  // below the wave's first scale; group h of the loads takes the row-block slots h and
  // h + 2 (one matrix per instruction).
  auto issue_scales = [&](const Unit& c, bool on) __attribute__((always_inline)) {
    const int wstart = (wave * c.steps * 8) & ~15;
#pragma unroll
    for (int i = 0; i < kSeqScaleLoads; ++i) {
      const int h = i / (kSeqScaleLoads / 2);
      const int f = (i % (kSeqScaleLoads / 2)) * 64 + lane;
      const int ri = (f * c.spr_recip) >> 16;  // f / spr (exact for f < 192, spr <= 24)
      const int piece = f - ri * c.spr;
      const int slot = h + 2 * (ri >> 4);
      const int row = (c.rb0 + (slot >> c.gated)) * 16 + (ri & 15);
      const int pofs = wstart + piece * 16;
      const int ok = (int)on & (int)(ri < 32) & (int)(slot < c.nrb) & (int)(row < c.n) & (int)(pofs < c.row_sbytes);
      sreg[i] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(h ? c.bs1 : c.bs0, (row * c.row_sbytes + pofs) & -ok, 0, 0));
    }
  };
  auto store_scales = [&](const Unit& c) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < kSeqScaleLoads; ++i) {
      const int h = i / (kSeqScaleLoads / 2);
      const int f = (i % (kSeqScaleLoads / 2)) * 64 + lane;
      const int ri = (f * c.spr_recip) >> 16;
      const int piece = f - ri * c.spr;
      const int slot = h + 2 * (ri >> 4);
      if (ri < 32) sarea[(slot * 16 + (ri & 15)) * c.spr + piece] = sreg[i];
    }
  };

  float4_t acc[RP];
#pragma unroll
  for (int r = 0; r < RP; ++r) acc[r] = (float4_t){0.f, 0.f, 0.f, 0.f};
  int finished = 0;  // units this workgroup has finished: the parity of the parked tiles

  // What an epilogue step with an input (a bias, a residual) adds to this thread's outputs
  // of the unit: loaded with the unit's scales, long before the unit ends, so that the end
  // of a unit issues no load.  A thread owns the outputs o = tid and tid + 512 of the
  // unit's 4 x 256 (gated: 2 x 256).
  constexpr int NOUT = RP * 256 / 512;
  float epin[NOUT][TLHIP_MAX_EPILOGUE_OPS];
  auto output_of = [&](const Unit& c, int i, int& b, int& m, int& col) __attribute__((always_inline)) {
    const int o = tid + i * 512;
    b = o >> 8;
    m = (o & 255) >> 4;
    col = (c.rb0 + b) * 16 + (o & 15);
  };
  auto issue_epilogue_inputs = [&](const Unit& c, bool on) __attribute__((always_inline)) {
    const SeqProblem& Q = table[c.pi];
    const char* dummy = (const char*)lds_pointer(&Q.x);
#pragma unroll
    for (int op = 0; op < TLHIP_MAX_EPILOGUE_OPS; ++op) {
      const int kind = lds_word(&Q.epi.kind[op]);
      const bool f16 = lds_word(&Q.epi.input_dtype[op]) == TLHIP_F16;
      const char* base = (const char*)lds_pointer(&Q.epi.input[op]);
      const bool has = on && op < lds_word(&Q.epi.n_ops) && (kind == TLHIP_EPI_BIAS || kind == TLHIP_EPI_BINARY) && base != nullptr;
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        int b, m, col;
        output_of(c, i, b, m, col);
        const bool ok = has && b < (c.nrb >> c.gated) && col < c.n && m < mrows;
        const int64_t at = kind == TLHIP_EPI_BIAS ? (int64_t)col : (int64_t)m * c.n + col;
        const char* p = ok ? base + at * (f16 ? 2 : 4) : dummy;
        // one 2-byte load either way (f32: the two halves would need two; a 4-byte load of an
        // f16 element could cross the end of its buffer), so both element types cost one load
        if (f16) epin[i][op] = (float)*as_global<const _Float16>(p);
        else epin[i][op] = *as_global<const float>((const void*)((uintptr_t)p & ~(uintptr_t)3));
      }
    }
  };

  // End of a unit: park, one barrier, every thread combines and stores its outputs; then
  // the unit is counted.  No load is issued here and the stores are two per thread under
  // the lane mask only: the number of memory operations between the next unit's first loads
  // (already in flight) and their use must be (nearly) the same on every path, or the
  // compiler has to wait for all of them.
  auto finish = [&](const Unit& c) __attribute__((always_inline)) {
    float* buf = parked + (finished & 1) * (W * RP * 256);
    ++finished;
#pragma unroll
    for (int r = 0; r < RP; ++r) {
#pragma unroll
      for (int q = 0; q < 4; ++q) buf[(wave * RP + r) * 256 + (4 * g + q) * 16 + nl] = acc[r][q];
      acc[r] = (float4_t){0.f, 0.f, 0.f, 0.f};
    }
    lds_barrier();
    const SeqProblem& Q = table[c.pi];
    char* y = (char*)const_cast<void*>(lds_pointer(&Q.y));
    const int y_dtype = lds_word(&Q.y_dtype);
    const float alpha = __builtin_bit_cast(float, lds_word(&Q.alpha));
    const int n_ops = lds_word(&Q.epi.n_ops);
    const int gated = c.gated;
    float v[NOUT];
    bool valid[NOUT];
    int64_t idx[NOUT];
#pragma unroll
    for (int i = 0; i < NOUT; ++i) {
      int b, m, col;
      output_of(c, i, b, m, col);
      const int e = (tid + i * 512) & 255;
      const int r0 = gated ? 2 * (b & 1) : b;  // b & 1: a slot that exists, also for an output that does not
      float s0 = 0.f, s1 = 0.f;
      for (int w = 0; w < W; ++w) {
        s0 += buf[(w * RP + r0) * 256 + e];
        s1 += buf[(w * RP + (r0 | 1)) * 256 + e];
      }
      valid[i] = b < (c.nrb >> gated) && col < c.n && m < mrows;
      idx[i] = (int64_t)m * c.n + col;
      v[i] = s0 * alpha;
#pragma unroll
      for (int op = 0; op < TLHIP_MAX_EPILOGUE_OPS; ++op) {
        if (op < n_ops) {
          const int kind = lds_word(&Q.epi.kind[op]);
          const int what = lds_word(&Q.epi.unary[op]);
          if (kind == TLHIP_EPI_BIAS) v[i] += epin[i][op];
          else if (kind == TLHIP_EPI_BINARY) v[i] = what == TLHIP_BINARY_ADD ? v[i] + epin[i][op] : (what == TLHIP_BINARY_SUB ? v[i] - epin[i][op] : v[i] * epin[i][op]);
          else if (kind == TLHIP_EPI_UNARY) v[i] = apply_unary(what, v[i]);
          else if (kind == TLHIP_EPI_CAST_F16) v[i] = (float)(_Float16)v[i];
        }
      }
      if (gated) v[i] *= s1 * alpha;
    }
    // A unit somebody waits for writes THROUGH to memory (agent-scope stores), waits until
    // the stores are acknowledged, and only then is counted: no write-back of the whole L2
    // (an agent-scope release fence cost each such unit tens of microseconds), and a
    // reader that has acquired at agent scope behind the count cannot see stale lines.
    const bool through = lds_word(&Q.signal) != 0;
    if (y_dtype == TLHIP_F16) {
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        const uint16_t bits = __builtin_bit_cast(uint16_t, (_Float16)v[i]);
        uint16_t TLHIP_GLOBAL* at = as_global<uint16_t>(y + idx[i] * 2);
        if (valid[i]) {
          if (through) __hip_atomic_store(at, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          else *at = bits;
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < NOUT; ++i) {
        float TLHIP_GLOBAL* at = as_global<float>(y + idx[i] * 4);
        if (valid[i]) {
          if (through) __hip_atomic_store(at, v[i], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          else *at = v[i];
        }
      }
    }
    if (through) {
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): every store of this wave is acknowledged
      __builtin_amdgcn_s_barrier();
    }
    if (a.counting && tid == 0)
      __hip_atomic_fetch_add(as_global<uint32_t>(&a.state->done[wg & (kSeqShards - 1)][0]), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  };

  auto consume = [&](int s, const Unit& c, int j) __attribute__((always_inline)) {
    const int st0 = wave * c.steps;
    if (j < c.steps && st0 + j < c.nsteps) {  // wave-uniform: a step beyond the wave's range or K adds nothing
#pragma unroll
      for (int q = 0; q < MQ; ++q) patch[(4 * q + xrow0) * RU + xunit] = permute_x_for_int4(rx[s][q]);
      half8_t xa[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) xa[t] = __builtin_bit_cast(half8_t, patch[nl * RU + 4 * t + g]);
      const int sbyte = ((st0 * 8) & 15) + j * 8;  // this step's scales inside the window
#pragma unroll
      for (int r = 0; r < RP; ++r) {
        if (r < c.nrb) {
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
    }
  };

  // Unit by unit.  The ring always holds the first D steps of the current unit when its
  // steady loop starts: they were issued (with the unit's scales in front of them) either
  // by the previous unit's last D steps or, at the start and behind a wait, by a prologue
  // of the same instructions, so the counters of loads in flight are the same either way.
  // A unit's steps are padded to a multiple of D; a padding step loads at offset 0 and
  // computes nothing.
  Unit cu, cn;
  enter(cu, 0);
  uint32_t waited = 0;  // units known to be done (the largest threshold waited for)
  bool prologue = true;
  while (cu.live) {
    if (prologue) {
      const uint32_t need = (uint32_t)(cu.first_unit + a.fault);
      if (cu.wait && need > waited) {
        // every unit in front of this problem must be done: wave 0 polls, everybody meets
        if (wave == 0) {
          uint32_t seen = 0;
          for (uint32_t spin = 0; spin < a.spin_limit; ++spin) {
            // lanes 0..15 read a shard each; the sum over the wave, less what the launch started with
            uint32_t part = __hip_atomic_load(as_global<uint32_t>(&a.state->done[lane & (kSeqShards - 1)][0]), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (lane >= kSeqShards) part = 0;
#pragma unroll
            for (int d = 1; d < kSeqShards; d *= 2) part += __shfl_xor(part, d);
            seen = (uint32_t)__builtin_amdgcn_readfirstlane((int)part) - a.base;
            if (seen >= need) break;
            __builtin_amdgcn_s_sleep(32);  // about a microsecond: pollers in a tight loop slow the counting down
          }
          if (lane == 0) {
            *flag = seen >= need ? 1 : 0;
            if (seen < need) __hip_atomic_fetch_or(as_global<uint32_t>(&a.state->error), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
        lds_barrier();
        const bool gave_up = *flag == 0;
        lds_barrier();  // nobody rewrites the flag before everybody has read it
        if (gave_up) break;
        // No agent-scope acquire here: it invalidates the XCD's whole L2, which every other
        // workgroup streams through, and cost a waiting launch 13 us.  What the wait orders
        // are this problem's activation loads, and those are agent-scope loads themselves.
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
        waited = need;
      }
      // the same memory operations in the same order as a unit's last D steps and its end
      // issue for the next unit (scales, D steps, the end's stores, epilogue inputs): the
      // counts of operations in flight then agree wherever the two paths meet
      issue_scales(cu, true);
#pragma unroll
      for (int s = 0; s < D; ++s) issue(s, cu, s, true);
      issue_epilogue_inputs(cu, true);
    }
    store_scales(cu);
    for (int j = 0; j + D < cu.steps_p; j += D) {
#pragma unroll
      for (int s = 0; s < D; ++s) {
        consume(s, cu, j + s);
        issue(s, cu, j + s + D, true);
      }
    }
    // the last D steps, with the next unit's first loads behind them (unless it has to wait)
    enter(cn, cu.i + 1);
    if (!cn.live) cn = cu, cn.live = 0;
    const bool next_on = cn.live && !(cn.wait && (uint32_t)(cn.first_unit + a.fault) > waited);
    issue_scales(cn, next_on);
#pragma unroll
    for (int s = 0; s < D; ++s) {
      consume(s, cu, cu.steps_p - D + s);
      issue(s, cn, s, next_on);
    }
    finish(cu);
    issue_epilogue_inputs(cn, next_on);  // behind finish: it reads the current unit's
    prologue = cn.live && !next_on;
    cu = cn;
  }
}

}  // namespace
}  // namespace tlhip
