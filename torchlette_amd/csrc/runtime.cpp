// Runtime half of the C ABI: device selection, memory, streams, events, the
// per-thread error string and the dispatch counters.  It plays the part the
// WebGPU device/queue plays for the reference backend
// (src/backend/webgpu/gpu-context.ts): ops enqueue on one in-order stream and
// only a read waits.
#include <atomic>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_map>
#include <unordered_set>

#include "common.h"

namespace tlhip {

namespace {
thread_local char g_error[512] = "";
std::mutex g_mutex;
bool g_init = false;
int g_device = -1;
hipStream_t g_stream = nullptr;
hipDeviceProp_t g_props;

std::atomic<uint64_t> g_gemv_dispatches{0};
std::atomic<uint64_t> g_gemm_dispatches{0};
std::atomic<uint64_t> g_dequant_dispatches{0};
std::atomic<uint64_t> g_autotune_runs{0};
std::atomic<uint64_t> g_tuning_entries_loaded{0};
}  // namespace

int set_error(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

void clear_error() { g_error[0] = '\0'; }

bool is_initialised() { return g_init; }

hipStream_t resolve_stream(tlhip_stream_t s) { return s ? static_cast<hipStream_t>(s) : g_stream; }

constexpr size_t kMlpScratchBytes = (size_t)2 << 20;  // 2 x 16 rows x 32768 f16

namespace {
// One workspace per stream.  A captured graph has the pointers of its capture stream's
// workspace baked into its kernel arguments, so the workspace outlives the stream for as
// long as a graph captured on it is alive: `graphs` counts those, `stream_alive` says
// whether tlhip_stream_destroy has been called.
struct SplitWorkspace {
  float* workspace;
  int* counters;
  uint32_t seq_base;  // what the unit counters of the stream's sequence launches add up to
  int graphs;
  bool stream_alive;
};
std::mutex g_ws_mutex;
std::unordered_map<hipStream_t, SplitWorkspace> g_workspaces;
struct GraphRecord {
  hipStream_t stream;  // the capture stream
  bool holds_workspace;  // counted in that stream's SplitWorkspace::graphs
};
std::unordered_map<hipGraphExec_t, GraphRecord> g_graphs;  // live graphs
std::unordered_set<hipStream_t> g_live_streams;            // the library stream and tlhip_stream_create's

void free_workspaces() {
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  for (auto& kv : g_graphs) (void)hipGraphExecDestroy(kv.first);  // graphs first: they reference the workspaces
  g_graphs.clear();
  for (auto& kv : g_workspaces) {
    (void)hipFree(kv.second.workspace);
    (void)hipFree(kv.second.counters);
  }
  g_workspaces.clear();
}

// Caller holds g_ws_mutex.
void release_if_unused(hipStream_t stream) {
  auto it = g_workspaces.find(stream);
  if (it == g_workspaces.end() || it->second.stream_alive || it->second.graphs > 0) return;
  (void)hipFree(it->second.workspace);
  (void)hipFree(it->second.counters);
  g_workspaces.erase(it);
}

void free_workspace_of(hipStream_t stream) {
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_workspaces.find(stream);
  if (it == g_workspaces.end()) return;
  it->second.stream_alive = false;
  release_if_unused(stream);
}
}  // namespace

int split_workspace(hipStream_t stream, float** workspace, int** counters) {
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto it = g_workspaces.find(stream);
  if (it == g_workspaces.end()) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    TLHIP_CHECK_HIP(hipStreamIsCapturing(stream, &status));
    if (status != hipStreamCaptureStatusNone)
      return set_error(TLHIP_ERR_STATE,
                       "split-K workspace of this stream does not exist yet and cannot be created during "
                       "capture: run the same call once on this stream before capturing");
    SplitWorkspace w{nullptr, nullptr, 0, 0, true};
    // + kMlpScratchBytes behind the workspace proper: the gate and up projections of
    // tlhip_mlp_decode's three-launch form (nobody else indexes past kSplitWorkspaceFloats)
    TLHIP_CHECK_HIP(hipMalloc((void**)&w.workspace, kSplitWorkspaceFloats * sizeof(float) + kMlpScratchBytes));
    // + 512 words behind the counters: the state of sequence launches on this stream
    hipError_t e = hipMalloc((void**)&w.counters, (kSplitCounters + 512) * sizeof(int));
    // on the stream that will use them (not capturing: checked above), so the clear is
    // ordered in front of the first launch whatever the stream's flags are
    if (e == hipSuccess) e = hipMemsetAsync(w.counters, 0, (kSplitCounters + 512) * sizeof(int), stream);
    if (e != hipSuccess) {
      (void)hipFree(w.workspace);
      if (w.counters) (void)hipFree(w.counters);
      return set_error(TLHIP_ERR_DEVICE, "split-K counters: %s", hipGetErrorString(e));
    }
    it = g_workspaces.emplace(stream, w).first;
  }
  *workspace = it->second.workspace;
  *counters = it->second.counters;
  return TLHIP_OK;
}

// 2 MiB of the stream's own behind its split-K workspace (gemv_seq.hip: the gate and up
// outputs of the MLP block between its launches).
int mlp_scratch(hipStream_t stream, void** scratch, size_t* bytes) {
  float* workspace = nullptr;
  int* counters = nullptr;
  const int rc = split_workspace(stream, &workspace, &counters);
  if (rc) return rc;
  *scratch = workspace + kSplitWorkspaceFloats;
  *bytes = kMlpScratchBytes;
  return TLHIP_OK;
}

// The device state of sequence launches on `stream` (gemv_seq.hip): 512 words behind the
// stream's split-K counters, and the host's running sum of its unit counters.
int sequence_state(hipStream_t stream, void** state, uint32_t** base) {
  float* workspace = nullptr;
  int* counters = nullptr;
  const int rc = split_workspace(stream, &workspace, &counters);
  if (rc) return rc;
  *state = counters + kSplitCounters;
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  *base = &g_workspaces.find(stream)->second.seq_base;  // the map's nodes do not move
  return TLHIP_OK;
}

namespace {
thread_local bool t_prepare_mode = false;
std::mutex g_lds_mutex;
std::unordered_set<const void*> g_lds_raised;

// Raises fn's dynamic-LDS limit to what the hardware leaves next to its static LDS, once.
int ensure_max_lds(const void* fn) {
  std::lock_guard<std::mutex> lock(g_lds_mutex);
  if (g_lds_raised.count(fn)) return TLHIP_OK;
  hipFuncAttributes attr;
  TLHIP_CHECK_HIP(hipFuncGetAttributes(&attr, fn));
  const int limit = 160 * 1024 - (int)attr.sharedSizeBytes;
  TLHIP_CHECK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, limit));
  g_lds_raised.insert(fn);
  return TLHIP_OK;
}
}  // namespace

bool prepare_mode() { return t_prepare_mode; }

int launch_kernel(const void* fn, dim3 grid, dim3 block, void** args, size_t lds_bytes, hipStream_t stream) {
  if (t_prepare_mode) return ensure_max_lds(fn);
  if (lds_bytes > 64 * 1024) {
    // already raised at tlhip_init; this is a set lookup
    const int rc = ensure_max_lds(fn);
    if (rc) return rc;
  }
  TLHIP_CHECK_HIP(hipLaunchKernel(fn, grid, block, args, lds_bytes, stream));
  return TLHIP_OK;
}

int prepare_gemv_seq_kernels();  // gemv_seq.hip

int prepare_all_kernels() {
  t_prepare_mode = true;
  int rc = prepare_gemv_kernels();
  if (!rc) rc = prepare_gemv_mfma_kernels();
  if (!rc) rc = prepare_gemv_xreg_kernels();
  if (!rc) rc = prepare_gemv_wave_kernels();
  if (!rc) rc = prepare_gemv_seq_kernels();
  if (!rc) rc = prepare_gemm_kernels();
  if (!rc) rc = prepare_gemm_direct_kernels();
  t_prepare_mode = false;
  return rc;
}

int problem_scratch(const Problem& p, hipStream_t stream, float** workspace, int** counters) {
  if (p.scratch) {
    *workspace = p.scratch->tiles;
    *counters = p.scratch->counters;
    return TLHIP_OK;
  }
  return split_workspace(stream, workspace, counters);
}

int device_cu_count() { return g_init ? g_props.multiProcessorCount : 0; }
int device_index() { return g_init ? g_device : -1; }

void count_gemv_dispatch() { g_gemv_dispatches++; }
void count_gemm_dispatch() { g_gemm_dispatches++; }
void count_dequant_dispatch() { g_dequant_dispatches++; }
void count_autotune_run() { g_autotune_runs++; }
void count_tuning_entries_loaded(int n) { g_tuning_entries_loaded += (uint64_t)(n > 0 ? n : 0); }

}  // namespace tlhip

using namespace tlhip;

extern "C" {

const char* tlhip_last_error(void) { return g_error; }

int tlhip_init(int device_index) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_init) {
    if (device_index == g_device) return TLHIP_OK;
    return set_error(TLHIP_ERR_STATE, "tlhip_init: already initialised on device %d", g_device);
  }
  int count = 0;
  hipError_t e = hipGetDeviceCount(&count);
  if (e != hipSuccess || count == 0) {
    return set_error(TLHIP_ERR_DEVICE, "tlhip_init: no HIP device available (%s); this backend has no CPU fallback",
                     e != hipSuccess ? hipGetErrorString(e) : "device count is 0");
  }
  if (device_index < 0 || device_index >= count)
    return set_error(TLHIP_ERR_INVALID, "tlhip_init: device index %d out of range [0,%d)", device_index, count);
  TLHIP_CHECK_HIP(hipSetDevice(device_index));
  TLHIP_CHECK_HIP(hipGetDeviceProperties(&g_props, device_index));
  if (strncmp(g_props.gcnArchName, "gfx950", 6) != 0) {
    return set_error(TLHIP_ERR_DEVICE, "tlhip_init: device %d is %s; this library carries gfx950 code only",
                     device_index, g_props.gcnArchName);
  }
  // Default priority only: mixed stream priorities are not used anywhere.
  TLHIP_CHECK_HIP(hipStreamCreateWithFlags(&g_stream, hipStreamNonBlocking));
  {
    std::lock_guard<std::mutex> ws_lock(g_ws_mutex);
    g_live_streams.insert(g_stream);
  }
  g_device = device_index;
  g_init = true;
  int rc = noalloc_setup(device_index);
  if (!rc) rc = prepare_all_kernels();
  if (rc) {
    (void)hipStreamDestroy(g_stream);
    g_stream = nullptr;
    g_init = false;
    g_device = -1;
    return rc;
  }
  count_tuning_entries_loaded(load_default_tuning());
  clear_error();
  return TLHIP_OK;
}

int tlhip_shutdown(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (!g_init) return TLHIP_OK;
  (void)hipStreamSynchronize(g_stream);
  free_workspaces();
  {
    std::lock_guard<std::mutex> ws_lock(g_ws_mutex);
    g_live_streams.clear();
  }
  (void)hipStreamDestroy(g_stream);
  g_stream = nullptr;
  g_init = false;
  g_device = -1;
  {
    std::lock_guard<std::mutex> lds_lock(g_lds_mutex);
    g_lds_raised.clear();
  }
  return TLHIP_OK;
}

int tlhip_device_info(tlhip_device_info_t* out) {
  TLHIP_REQUIRE_INIT();
  if (!out) return set_error(TLHIP_ERR_INVALID, "tlhip_device_info: null output");
  memset(out, 0, sizeof(*out));
  strncpy(out->name, g_props.name, sizeof(out->name) - 1);
  strncpy(out->arch, g_props.gcnArchName, sizeof(out->arch) - 1);
  out->compute_units = g_props.multiProcessorCount;
  out->wavefront_size = g_props.warpSize;
  out->lds_bytes_per_block = (int32_t)g_props.sharedMemPerBlock;
  out->clock_khz = g_props.clockRate;
  out->memory_clock_khz = g_props.memoryClockRate;
  out->memory_bus_bits = g_props.memoryBusWidth;
  out->total_memory_bytes = (int64_t)g_props.totalGlobalMem;
  out->l2_bytes = (int64_t)g_props.l2CacheSize;
  return TLHIP_OK;
}

int tlhip_malloc(size_t bytes, void** out) {
  TLHIP_REQUIRE_INIT();
  if (!out) return set_error(TLHIP_ERR_INVALID, "tlhip_malloc: null output");
  *out = nullptr;
  if (bytes == 0) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipMalloc(out, bytes));
  return TLHIP_OK;
}

int tlhip_free(void* ptr) {
  TLHIP_REQUIRE_INIT();
  if (!ptr) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipFree(ptr));
  return TLHIP_OK;
}

int tlhip_memset(void* ptr, int value, size_t bytes, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (bytes == 0) return TLHIP_OK;
  // not into a graph: memset nodes have given wrong results on replays after the first
  hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
  TLHIP_CHECK_HIP(hipStreamIsCapturing(resolve_stream(stream), &status));
  if (status != hipStreamCaptureStatusNone)
    return set_error(TLHIP_ERR_STATE, "tlhip_memset: the stream is being captured; clear memory before the capture "
                                      "or with a kernel");
  TLHIP_CHECK_HIP(hipMemsetAsync(ptr, value, bytes, resolve_stream(stream)));
  return TLHIP_OK;
}

int tlhip_memcpy_h2d(void* dst, const void* host_src, size_t bytes, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (bytes == 0) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipMemcpyAsync(dst, host_src, bytes, hipMemcpyHostToDevice, resolve_stream(stream)));
  return TLHIP_OK;
}

int tlhip_memcpy_d2h(void* host_dst, const void* src, size_t bytes, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (bytes == 0) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipMemcpyAsync(host_dst, src, bytes, hipMemcpyDeviceToHost, resolve_stream(stream)));
  return TLHIP_OK;
}

int tlhip_memcpy_d2d(void* dst, const void* src, size_t bytes, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (bytes == 0) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, resolve_stream(stream)));
  return TLHIP_OK;
}

int tlhip_host_alloc(size_t bytes, void** out) {
  TLHIP_REQUIRE_INIT();
  if (!out) return set_error(TLHIP_ERR_INVALID, "tlhip_host_alloc: null output");
  TLHIP_CHECK_HIP(hipHostMalloc(out, bytes ? bytes : 1, hipHostMallocDefault));
  return TLHIP_OK;
}

int tlhip_host_free(void* host_ptr) {
  TLHIP_REQUIRE_INIT();
  if (!host_ptr) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipHostFree(host_ptr));
  return TLHIP_OK;
}

int tlhip_stream_create(tlhip_stream_t* out) {
  TLHIP_REQUIRE_INIT();
  if (!out) return set_error(TLHIP_ERR_INVALID, "tlhip_stream_create: null output");
  hipStream_t s;
  TLHIP_CHECK_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    g_live_streams.insert(s);
    // a handle value can come back after its stream was destroyed: a workspace that live
    // graphs of the old stream keep is this stream's workspace again
    auto it = g_workspaces.find(s);
    if (it != g_workspaces.end()) it->second.stream_alive = true;
  }
  *out = s;
  return TLHIP_OK;
}

int tlhip_stream_destroy(tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (!stream) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipStreamSynchronize(static_cast<hipStream_t>(stream)));
  free_workspace_of(static_cast<hipStream_t>(stream));
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    g_live_streams.erase(static_cast<hipStream_t>(stream));
  }
  TLHIP_CHECK_HIP(hipStreamDestroy(static_cast<hipStream_t>(stream)));
  return TLHIP_OK;
}

int tlhip_stream_synchronize(tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  TLHIP_CHECK_HIP(hipStreamSynchronize(resolve_stream(stream)));
  return TLHIP_OK;
}

int tlhip_event_create(tlhip_event_t* out) {
  TLHIP_REQUIRE_INIT();
  if (!out) return set_error(TLHIP_ERR_INVALID, "tlhip_event_create: null output");
  hipEvent_t e;
  TLHIP_CHECK_HIP(hipEventCreate(&e));
  *out = e;
  return TLHIP_OK;
}

int tlhip_event_destroy(tlhip_event_t ev) {
  TLHIP_REQUIRE_INIT();
  if (!ev) return TLHIP_OK;
  TLHIP_CHECK_HIP(hipEventDestroy(static_cast<hipEvent_t>(ev)));
  return TLHIP_OK;
}

int tlhip_event_record(tlhip_event_t ev, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  TLHIP_CHECK_HIP(hipEventRecord(static_cast<hipEvent_t>(ev), resolve_stream(stream)));
  return TLHIP_OK;
}

int tlhip_event_synchronize(tlhip_event_t ev) {
  TLHIP_REQUIRE_INIT();
  TLHIP_CHECK_HIP(hipEventSynchronize(static_cast<hipEvent_t>(ev)));
  return TLHIP_OK;
}

int tlhip_event_elapsed_us(tlhip_event_t start, tlhip_event_t stop, double* out_us) {
  TLHIP_REQUIRE_INIT();
  if (!out_us) return set_error(TLHIP_ERR_INVALID, "tlhip_event_elapsed_us: null output");
  float ms = 0.f;
  TLHIP_CHECK_HIP(hipEventElapsedTime(&ms, static_cast<hipEvent_t>(start), static_cast<hipEvent_t>(stop)));
  *out_us = (double)ms * 1000.0;
  return TLHIP_OK;
}

int tlhip_graph_begin_capture(tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  TLHIP_CHECK_HIP(hipStreamBeginCapture(resolve_stream(stream), hipStreamCaptureModeThreadLocal));
  return TLHIP_OK;
}

int tlhip_graph_end_capture(tlhip_stream_t stream, tlhip_graph_t* out) {
  TLHIP_REQUIRE_INIT();
  if (!out) return set_error(TLHIP_ERR_INVALID, "tlhip_graph_end_capture: null output");
  hipStream_t s = resolve_stream(stream);
  hipGraph_t graph = nullptr;
  TLHIP_CHECK_HIP(hipStreamEndCapture(s, &graph));
  hipGraphExec_t exec = nullptr;
  hipError_t e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
  (void)hipGraphDestroy(graph);
  if (e != hipSuccess) return set_error(TLHIP_ERR_DEVICE, "hipGraphInstantiate failed: %s", hipGetErrorString(e));
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_workspaces.find(s);
    g_graphs[exec] = GraphRecord{s, it != g_workspaces.end()};
    if (it != g_workspaces.end()) it->second.graphs++;
  }
  *out = exec;
  return TLHIP_OK;
}

int tlhip_graph_launch(tlhip_graph_t graph, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  if (!graph) return set_error(TLHIP_ERR_INVALID, "tlhip_graph_launch: null graph");
  hipStream_t s = resolve_stream(stream);
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_graphs.find(static_cast<hipGraphExec_t>(graph));
    if (it == g_graphs.end()) return set_error(TLHIP_ERR_INVALID, "tlhip_graph_launch: unknown or destroyed graph");
    // the captured kernels use the capture stream's K-slice workspace; on another stream a
    // replay could run next to that stream's own launches on the same tiles and counters
    if (it->second.stream != s)
      return set_error(TLHIP_ERR_INVALID, "tlhip_graph_launch: a graph replays on the stream it was captured on");
  }
  TLHIP_CHECK_HIP(hipGraphLaunch(static_cast<hipGraphExec_t>(graph), s));
  return TLHIP_OK;
}

int tlhip_graph_destroy(tlhip_graph_t graph) {
  TLHIP_REQUIRE_INIT();
  if (!graph) return TLHIP_OK;
  hipGraphExec_t exec = static_cast<hipGraphExec_t>(graph);
  hipStream_t origin = nullptr;
  bool held = false;
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    auto it = g_graphs.find(exec);
    if (it == g_graphs.end()) return TLHIP_OK;  // idempotent, like destroy() in the reference
    origin = it->second.stream;
    held = it->second.holds_workspace;
    g_graphs.erase(it);
  }
  // a replay may still be in flight on the capture stream (the library stream is never destroyed
  // before shutdown; a caller's stream that is already gone has been synchronised by its destroy)
  bool alive;
  {
    std::lock_guard<std::mutex> lock(g_ws_mutex);
    alive = g_live_streams.count(origin) != 0;
  }
  if (alive) (void)hipStreamSynchronize(origin);
  TLHIP_CHECK_HIP(hipGraphExecDestroy(exec));
  std::lock_guard<std::mutex> lock(g_ws_mutex);
  auto w = g_workspaces.find(origin);
  if (held && w != g_workspaces.end() && w->second.graphs > 0) {
    w->second.graphs--;
    release_if_unused(origin);
  }
  return TLHIP_OK;
}

uint64_t tlhip_counter(const char* name) {
  if (!name) return 0;
  if (!strcmp(name, "quant_gemv_dispatches")) return g_gemv_dispatches.load();
  if (!strcmp(name, "quant_gemm_dispatches")) return g_gemm_dispatches.load();
  if (!strcmp(name, "dequant_dispatches")) return g_dequant_dispatches.load();
  if (!strcmp(name, "autotune_runs")) return g_autotune_runs.load();
  if (!strcmp(name, "tuning_entries_loaded")) return g_tuning_entries_loaded.load();
  return 0;
}

int tlhip_counters_reset(void) {
  g_gemv_dispatches = 0;
  g_gemm_dispatches = 0;
  g_dequant_dispatches = 0;
  g_autotune_runs = 0;
  return TLHIP_OK;
}

}  // extern "C"
