// Host side of the sequence launch (gemv_seq_kernel.h): tlhip_gemv_sequence,
// tlhip_mlp_decode, tlhip_sequence_status.
#include <atomic>

#include "gemv_seq_kernel.h"

namespace tlhip {
int sequence_state(hipStream_t stream, void** state, uint32_t** base);  // runtime.cpp

namespace {

constexpr int kSeqWaves = 8;
constexpr uint32_t kSeqSpinLimit = 1u << 22;  // polls of about 0.1 us each: a wait gives up after roughly half a second

std::atomic<int> g_seq_fault{0};
std::atomic<uint32_t> g_seq_spin_limit{kSeqSpinLimit};

const void* seq_fn(int mq) {
  switch (mq) {
    case 1: return (const void*)gemv_seq_kernel<1, 2>;
    case 2: return (const void*)gemv_seq_kernel<2, 2>;
    case 4: return (const void*)gemv_seq_kernel<4, 2>;
  }
  return nullptr;
}

size_t seq_lds_bytes() {
  return (size_t)kSeqWaves * (16 * 17 + kSeqScaleLoads * 64) * 16 + (size_t)2 * kSeqWaves * kSeqSlots * 1024 + 16 +
         sizeof(SeqProblem) * kSeqMaxProblems;
}

}  // namespace

int prepare_gemv_seq_kernels() {
  for (int mq : {1, 2, 4}) {
    const int rc = launch_kernel(seq_fn(mq), dim3(1), dim3(64), nullptr, 0, nullptr);
    if (rc) return rc;
  }
  return TLHIP_OK;
}

int mlp_scratch(hipStream_t stream, void** scratch, size_t* bytes);  // runtime.cpp

}  // namespace tlhip

using namespace tlhip;

extern "C" {

int tlhip_gemv_sequence(const tlhip_sequence_step_t* steps, int count, int x_dtype, int64_t m, float alpha,
                        tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  clear_error();
  if (!steps || count < 1 || count > kSeqMaxProblems)
    return set_error(TLHIP_ERR_INVALID, "gemv_sequence: 1..%d steps", kSeqMaxProblems);
  if (x_dtype != TLHIP_F16) return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: activations must be f16");
  if (m < 1 || m > 16) return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: M must be 1..16");
  int mq = 1;
  while (mq * 4 < m) mq *= 2;
  const int cus = device_cu_count() > 0 ? device_cu_count() : 256;
  SeqTable t;
  memset(&t, 0, sizeof t);
  t.count = count;
  t.m = (int)m;
  int64_t units = 0;
  int last_wait = -1;
  for (int i = 0; i < count; ++i)
    if (steps[i].wait) last_wait = i;
  for (int i = 0; i < count; ++i) {
    const tlhip_sequence_step_t& s = steps[i];
    Problem p;
    int rc = make_problem(&s.w, s.x, x_dtype, m, s.y, s.y_dtype, alpha, s.epilogue, &p, "gemv_sequence");
    if (rc) return rc;
    if (p.format != TLHIP_FMT_INT4_GROUPED || p.group_size != 32)
      return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: built for int4 weights with group size 32");
    if (p.k % 128 != 0 || p.n < 1) return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: K must be a multiple of 128 and N at least 1");
    const int64_t lim = (int64_t)1 << 31;
    if (p.n * (p.k / 2) >= lim || m * p.k * 2 >= lim)
      return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: weights and activations must each be below 2 GiB");
    SeqProblem& P = t.p[i];
    P.packed[0] = P.packed[1] = p.packed;
    P.scales[0] = P.scales[1] = p.scales;
    if (s.gated) {
      rc = validate_weight(&s.w_up, "gemv_sequence");
      if (rc) return rc;
      if (s.w_up.format != s.w.format || s.w_up.group_size != s.w.group_size || s.w_up.n != s.w.n || s.w_up.k != s.w.k)
        return set_error(TLHIP_ERR_INVALID, "gemv_sequence: the two weights of a gated step must have the same format and shape");
      P.packed[1] = s.w_up.packed;
      P.scales[1] = s.w_up.scales;
    }
    if (i == 0 && s.wait) return set_error(TLHIP_ERR_INVALID, "gemv_sequence: the first step has nothing to wait for");
    // Only activations may be an earlier step's output (they are loaded at agent scope
    // behind the wait); bias and binary inputs are loaded early and through the caches.
    for (int op = 0; op < p.epi.n_ops; ++op) {
      if (!p.epi.input[op]) continue;
      const bool binary = p.epi.kind[op] == TLHIP_EPI_BINARY;
      const char* i0 = (const char*)p.epi.input[op];
      const char* i1 = i0 + (size_t)(binary ? m * p.n : p.n) * (p.epi.input_dtype[op] == TLHIP_F16 ? 2 : 4);
      for (int j = 0; j < i; ++j) {
        const char* y0 = (const char*)steps[j].y;
        const char* y1 = y0 + (size_t)m * (size_t)steps[j].w.n * (steps[j].y_dtype == TLHIP_F16 ? 2 : 4);
        if (y0 && i0 < y1 && y0 < i1)
          return set_error(TLHIP_ERR_INVALID, "gemv_sequence: an epilogue input of step %d overlaps the output of step %d of the "
                                              "same launch (only activations may be an earlier step's output)", i, j);
      }
    }
    P.x = p.x;
    P.y = p.y;
    P.packed_bytes = (uint32_t)(p.n * (p.k / 2));
    P.scales_bytes = (uint32_t)(p.n * (p.k / 32) * 2);
    P.x_bytes = (uint32_t)(m * p.k * 2);
    P.n = (int)p.n;
    P.kb = (int)(p.k / 2);
    P.nsteps = (int)(p.k / 128);
    P.steps = (P.nsteps + kSeqWaves - 1) / kSeqWaves;
    P.spr = (((P.steps & 1) ? 8 : 0) + P.steps * 8 + 15) / 16;
    if (32 * P.spr > (kSeqScaleLoads / 2) * 64)
      return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: K above 12288 (the scales of a wave's K range are loaded up front)");
    if ((p.k / 16) % 16 != 0)
      return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: K must be a multiple of 256");
    P.spr_recip = (65536 + P.spr - 1) / P.spr;
    P.first_unit = (int)units;
    P.gated = s.gated ? 1 : 0;
    P.wait = s.wait ? 1 : 0;
    P.signal = i < last_wait ? 1 : 0;
    P.y_dtype = s.y_dtype;
    P.alpha = alpha;
    P.epi = p.epi;
    // Row blocks per unit: as few as still give every CU a unit (a problem of 256 row blocks
    // on 256 CUs goes one block to a unit; more blocks per unit share the unit's activation
    // loads), at most what the kernel's four slots hold (a gated row block takes two).
    const int64_t nblocks = (p.n + 15) / 16;
    int64_t per_unit = (nblocks + cus - 1) / cus;
    const int64_t most = s.gated ? 2 : 4;
    if (per_unit > most) per_unit = most;
    P.nrb = (int)(s.gated ? 2 * per_unit : per_unit);
    units += (nblocks + per_unit - 1) / per_unit;
  }
  if (units >= ((int64_t)1 << 30)) return set_error(TLHIP_ERR_UNSUPPORTED, "gemv_sequence: too many rows");
  t.total_units = (int)units;
  t.fault = g_seq_fault.load();
  t.counting = last_wait >= 0 ? 1 : 0;
  hipStream_t hs = resolve_stream(stream);
  void* state = nullptr;
  uint32_t* base = nullptr;  // host copy of what the stream's unit counters add up to
  int rc = sequence_state(hs, &state, &base);
  if (rc) return rc;
  t.state = (SeqState*)state;
  if (t.counting) {
    // the counters' value is baked into the launch: a captured launch would replay with a stale one
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    TLHIP_CHECK_HIP(hipStreamIsCapturing(hs, &status));
    if (status != hipStreamCaptureStatusNone)
      return set_error(TLHIP_ERR_STATE, "gemv_sequence: a sequence with a waiting step cannot be captured into a graph");
    t.base = *base;
    *base += (uint32_t)units;
  }
  t.spin_limit = g_seq_spin_limit.load();
  // Every workgroup must be resident (a unit may wait for units of other workgroups): one
  // per CU (the kernel's LDS lets no second one in), and never more than there are units.
  const int grid = (int)(units < cus ? units : cus);
  const void* fn = seq_fn(mq);
  void* args[] = {(void*)&t};
  rc = launch_kernel(fn, dim3(grid), dim3(kSeqWaves * 64), args, seq_lds_bytes(), hs);
  if (rc) return rc;
  TLHIP_CHECK_HIP(hipGetLastError());
  for (int i = 0; i < count; ++i) count_gemv_dispatch();
  return TLHIP_OK;
}

// The MLP block as ONE sequence launch: a gated step (both projections of a row block in one
// unit, act(gate) * up written as f16) and the down projection waiting for it.
static int mlp_one_launch(const tlhip_qweight_t* gate, const tlhip_qweight_t* up, const tlhip_qweight_t* down, int unary,
                          const void* x, int x_dtype, int64_t m, void* h, void* y, int y_dtype,
                          const tlhip_epilogue_t* down_epilogue, tlhip_stream_t stream) {
  tlhip_epilogue_t act;
  memset(&act, 0, sizeof act);
  act.n_ops = 1;
  act.ops[0].kind = TLHIP_EPI_UNARY;
  act.ops[0].unary = unary;
  tlhip_sequence_step_t steps[2];
  memset(steps, 0, sizeof steps);
  steps[0].w = *gate;
  steps[0].w_up = *up;
  steps[0].gated = 1;
  steps[0].x = x;
  steps[0].y = h;
  steps[0].y_dtype = TLHIP_F16;  // the down projection's activation type
  steps[0].epilogue = &act;
  steps[1].w = *down;
  steps[1].x = h;
  steps[1].y = y;
  steps[1].y_dtype = y_dtype;
  steps[1].epilogue = down_epilogue;
  steps[1].wait = 1;
  return tlhip_gemv_sequence(steps, 2, x_dtype, m, 1.0f, stream);
}

// One call for the block, whichever way is faster.  Measured on MI355X at 1..16 rows the
// three launches the model issues (gate and up grouped on the shared activations, the gated
// multiply, down) take 23-33 us at 4096 -> 12288 -> 4096 and the sequence launch 42-50 us,
// so the three launches are what runs; TLHIP_MLP_ONE_LAUNCH=1 selects the sequence launch.
// Between its launches the gate and up outputs live in 2 MiB of the stream's workspace.
int tlhip_mlp_decode(const tlhip_qweight_t* gate, const tlhip_qweight_t* up, const tlhip_qweight_t* down, int unary,
                     const void* x, int x_dtype, int64_t m, void* h, void* y, int y_dtype,
                     const tlhip_epilogue_t* down_epilogue, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  clear_error();
  if (!gate || !up || !down || !h) return set_error(TLHIP_ERR_INVALID, "mlp_decode: null argument");
  if (down->k != gate->n) return set_error(TLHIP_ERR_INVALID, "mlp_decode: down.K must equal gate.N");
  if (up->n != gate->n || up->k != gate->k || up->format != gate->format || up->group_size != gate->group_size)
    return set_error(TLHIP_ERR_INVALID, "mlp_decode: gate and up must have the same format and shape");
  if (y_dtype != TLHIP_F16 && y_dtype != TLHIP_F32) return set_error(TLHIP_ERR_INVALID, "mlp_decode: y must be f16 or f32");
  if (x_dtype != TLHIP_F16) return set_error(TLHIP_ERR_UNSUPPORTED, "mlp_decode: activations must be f16");
  if (m < 1 || m > 16) return set_error(TLHIP_ERR_INVALID, "mlp_decode: M must be 1..16, got %lld", (long long)m);
  static const bool one_launch = [] {
    const char* e = getenv("TLHIP_MLP_ONE_LAUNCH");
    return e && e[0] == '1';
  }();
  if (one_launch) return mlp_one_launch(gate, up, down, unary, x, x_dtype, m, h, y, y_dtype, down_epilogue, stream);
  void* scratch = nullptr;
  size_t scratch_bytes = 0;
  int rc = mlp_scratch(resolve_stream(stream), &scratch, &scratch_bytes);
  if (rc) return rc;
  const size_t one = (size_t)m * (size_t)gate->n * sizeof(_Float16);
  if (2 * one > scratch_bytes) return mlp_one_launch(gate, up, down, unary, x, x_dtype, m, h, y, y_dtype, down_epilogue, stream);
  tlhip_gemv_problem_t both[2];
  memset(both, 0, sizeof both);
  both[0].w = *gate;
  both[0].x = x;
  both[0].y = scratch;
  both[1].w = *up;
  both[1].x = x;
  both[1].y = (char*)scratch + one;
  rc = tlhip_gemv_grouped_rows(both, 2, x_dtype, m, TLHIP_F16, 1.0f, stream);
  if (rc) return rc;
  rc = tlhip_gated_mul(unary, both[0].y, both[1].y, TLHIP_F16, h, m * gate->n, stream);
  if (rc) return rc;
  return tlhip_gemv(down, h, TLHIP_F16, m, y, y_dtype, 1.0f, down_epilogue, stream);
}

int tlhip_sequence_status(tlhip_stream_t stream, int* error) {
  TLHIP_REQUIRE_INIT();
  clear_error();
  if (!error) return set_error(TLHIP_ERR_INVALID, "sequence_status: null argument");
  hipStream_t hs = resolve_stream(stream);
  void* state = nullptr;
  uint32_t* base = nullptr;
  const int rc = sequence_state(hs, &state, &base);
  if (rc) return rc;
  uint32_t err = 0;
  TLHIP_CHECK_HIP(hipMemcpyAsync(&err, &((SeqState*)state)->error, sizeof err, hipMemcpyDeviceToHost, hs));
  TLHIP_CHECK_HIP(hipStreamSynchronize(hs));
  *error = (int)err;
  if (err) {
    // a wait expired: some workgroups left early, so the counters are behind the host's sum
    TLHIP_CHECK_HIP(hipMemsetAsync(state, 0, sizeof(SeqState), hs));
    TLHIP_CHECK_HIP(hipStreamSynchronize(hs));
    *base = 0;
    return set_error(TLHIP_ERR_DEVICE, "gemv_sequence: a wait for earlier steps of a launch expired; its results are incomplete");
  }
  return TLHIP_OK;
}

int tlhip_debug_sequence(int fault, uint32_t spin_limit) {
  g_seq_fault.store(fault ? 1 : 0);
  g_seq_spin_limit.store(spin_limit ? spin_limit : kSeqSpinLimit);
  return TLHIP_OK;
}

}  // extern "C"
