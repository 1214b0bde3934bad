// Internal declarations shared by the translation units of libtlhip.so.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "tlhip.h"

namespace tlhip {

// Per-thread error text behind tlhip_last_error().
int set_error(int code, const char* fmt, ...);
void clear_error();

bool is_initialised();
hipStream_t resolve_stream(tlhip_stream_t s);  // NULL -> library stream
int device_cu_count();
int device_index();  // the device tlhip_init selected, -1 before

#define TLHIP_CHECK_HIP(expr)                                                            \
  do {                                                                                   \
    hipError_t _e = (expr);                                                              \
    if (_e != hipSuccess)                                                                \
      return ::tlhip::set_error(TLHIP_ERR_DEVICE, "%s failed: %s", #expr, hipGetErrorString(_e)); \
  } while (0)

#define TLHIP_REQUIRE_INIT()                                                             \
  do {                                                                                   \
    if (!::tlhip::is_initialised())                                                      \
      return ::tlhip::set_error(TLHIP_ERR_STATE, "tlhip: not initialised (call tlhip_init)"); \
  } while (0)

// Epilogue as the kernels take it (by value, in kernel arguments).
struct DevEpilogue {
  int n_ops;
  int kind[TLHIP_MAX_EPILOGUE_OPS];
  int unary[TLHIP_MAX_EPILOGUE_OPS];
  int input_dtype[TLHIP_MAX_EPILOGUE_OPS];
  const void* input[TLHIP_MAX_EPILOGUE_OPS];
};

// The epilogue of the rows from m0 on of a problem with n columns: a binary step's [M,N]
// input starts m0 rows further, like the output.
inline DevEpilogue epilogue_from_row(DevEpilogue e, int64_t m0, int64_t n) {
  for (int i = 0; i < e.n_ops; ++i)
    if (e.kind[i] == TLHIP_EPI_BINARY && e.input[i])
      e.input[i] = (const char*)e.input[i] + m0 * n * (e.input_dtype[i] == TLHIP_F16 ? 2 : 4);
  return e;
}

// Prologue of the VALU decode GEMV (tlhip_prologue_t as the kernel takes it).
struct DevPrologue {
  int kind;
  int unary;
  float eps;
  const void* operand;
};

// Caller-provided device scratch for the kernels that combine partial results of
// several workgroups (instead of the library's per-stream workspace): `tile_floats`
// floats of partial tiles and `ncounters` arrival counters that are zero when the
// launch starts.
struct SplitScratch {
  float* tiles;
  int* counters;
  size_t tile_floats;
  int ncounters;
};

// Validated problem description handed to the launchers.
struct Problem {
  int format;
  int group_size;
  int64_t n, k, m;
  const void* packed;
  const void* scales;
  const void* x;
  int x_dtype;
  void* y;
  int y_dtype;
  float alpha;
  DevEpilogue epi;
  DevPrologue pro;  // kind NONE unless the entry point sets it
  const SplitScratch* scratch;  // null: the library's per-stream workspace
};

// Validation shared by every compute entry point.  Fills `p` on success.
int make_problem(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y,
                 int y_dtype, float alpha, const tlhip_epilogue_t* epilogue, Problem* p,
                 const char* who);
int validate_weight(const tlhip_qweight_t* w, const char* who);

// Launchers (each returns a TLHIP_* code; launch errors are reported).
int launch_dequant(const tlhip_qweight_t& w, float* out, hipStream_t stream);
bool gemv_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why);
int launch_gemv(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream);
bool gemv_group_compatible(const Problem* ps, int count, const tlhip_kernel_config_t& c, const char** why);
int launch_gemv_grouped(const Problem* ps, int count, const tlhip_kernel_config_t& c, hipStream_t stream);
bool gemv_mfma_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why);
int launch_gemv_mfma(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream);
bool gemv_mfma_group_applicable(const Problem* ps, int count, const tlhip_kernel_config_t& c, const char** why);
int launch_gemv_mfma_group(const Problem* ps, int count, const tlhip_kernel_config_t& c, hipStream_t stream);
bool gemv_xreg_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why);
int launch_gemv_xreg(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream);
// up to 4 problems that share activations, rows and shape class in one launch
bool gemv_xreg_group_applicable(const Problem* ps, int count, const tlhip_kernel_config_t& c, const char** why);
int launch_gemv_xreg_group(const Problem* ps, int count, const tlhip_kernel_config_t& c, hipStream_t stream);
bool gemv_wave_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why);
int launch_gemv_wave(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream);
// elementwise.hip: the steps of `ep` over a finished [M,N] output, in place, 8 columns a lane
bool epilogue_tail_applicable(const void* y, int64_t n);
int launch_epilogue_tail(void* y, int y_dtype, int64_t m, int64_t n, const DevEpilogue& ep, hipStream_t stream);
bool gemm_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why);
int launch_gemm(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream);
bool gemm_direct_config_applicable(const Problem& p, const tlhip_kernel_config_t& c, const char** why);
int launch_gemm_direct(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream);

// Device scratch for kernels that combine partial results of several workgroups:
// `kSplitWorkspaceFloats` floats plus `kSplitCounters` arrival counters that are
// zero whenever no launch is in flight.  One per stream, so launches on different
// streams never share it; created on the stream's first use, which must not
// happen while the stream is being captured.
constexpr size_t kSplitWorkspaceFloats = 8u << 20;  // 32 MiB
constexpr int kSplitCounters = 1 << 16;
int split_workspace(hipStream_t stream, float** workspace, int** counters);
// The scratch a launch of `p` combines its K slices through: the caller's, or the
// stream's own (created on first use).
int problem_scratch(const Problem& p, hipStream_t stream, float** workspace, int** counters);
inline size_t scratch_tile_floats(const Problem& p) { return p.scratch ? p.scratch->tile_floats : kSplitWorkspaceFloats; }
inline int scratch_counters(const Problem& p) { return p.scratch ? p.scratch->ncounters : kSplitCounters; }

// Kernel choice of the decode entry points (dispatch.cpp): the tuned winner for the
// problem if one is cached and applicable, else the heuristic default; never a
// prefill GEMM configuration.
tlhip_kernel_config_t select_gemv_config(const Problem& p);
int run_kernel_config(const Problem& p, const tlhip_kernel_config_t& c, hipStream_t stream);
// K slices across workgroups of a configuration (1 = it needs no scratch).
int config_k_slices(const tlhip_kernel_config_t& c);

// Imports the tuning file that ships with the library (dispatch.cpp); returns the number
// of entries added.
int load_default_tuning();
void count_tuning_entries_loaded(int n);

// Set-up of the entry point that allocates nothing (noalloc.hip): resolves the device
// address of its static scratch array for the current device.
int noalloc_setup(int device_index);

// Launch of a library kernel.  A kernel that takes more than 64 KiB of dynamic LDS needs its
// limit raised (hipFuncSetAttribute); that is done once per kernel, for every kernel of the
// library, at tlhip_init (prepare_all_kernels: each translation unit walks its own dispatch
// tables in "prepare mode", in which launch_kernel raises the limit and launches nothing),
// so that no launch, and nothing a caller captures into a graph, carries an attribute call.
int launch_kernel(const void* fn, dim3 grid, dim3 block, void** args, size_t lds_bytes, hipStream_t stream);
bool prepare_mode();
int prepare_all_kernels();
int prepare_gemv_kernels();       // gemv.hip (+ the per-format units)
int prepare_gemv_mfma_kernels();  // gemv_mfma.hip
int prepare_gemv_xreg_kernels();  // gemv_mfma_xreg.hip
int prepare_gemv_wave_kernels();  // gemv_wave.hip
int prepare_gemm_kernels();       // gemm_prefill.hip
int prepare_gemm_direct_kernels();  // gemm_direct.hip

// Counters.
void count_gemv_dispatch();
void count_gemm_dispatch();
void count_dequant_dispatch();
void count_autotune_run();

enum { VARIANT_GEMV = 0, VARIANT_GEMV_MFMA = 1, VARIANT_TILED = 2, VARIANT_TILED_DIRECT = 3, VARIANT_GEMV_XREG = 4, VARIANT_GEMV_WAVE = 5 };

}  // namespace tlhip
