// The decode GEMV for callers that cannot allocate device memory (code under HIP graph
// capture, tight serving loops, harnesses that forbid hipMalloc).
//
// tlhip_gemv combines the K slices of different workgroups through a workspace that the
// library allocates on a stream's first use.  tlhip_gemv_noalloc runs the same kernels
// with that workspace inside ONE file-scope device array of fixed size, so the call
// allocates nothing: no hipMalloc, no hipFree, no allocating library routine.  Every GPU
// holds its own copy of the array at its own address until the process ends; the address
// is resolved once per device at tlhip_init and host code uses that pointer only (the
// array's name is a host-side stand-in, not a device address).
//
// All calls on one GPU share the array and it keeps the last call's contents: the
// arrival counters a launch uses are cleared by a small fill kernel in front of it, the
// partial tiles are written before they are read.  Calls that overlap on one GPU
// (different streams, or a replaying graph next to eager calls) race.
#include "device_utils.h"

namespace tlhip {
int run_gemv_route(const Problem& p, hipStream_t stream);  // dispatch.cpp
int gemv_route_k_slices(const Problem& p);
namespace {

// Partial 16 x 16 f32 tiles, [row block][K slice][256], then one arrival counter per
// 16-row block.  4 MiB of tiles cover e.g. N = 16384 output rows with 4 K slices.
constexpr size_t kNoAllocTileFloats = 1u << 20;  // 4 MiB
constexpr int kNoAllocCounters = 4096;           // 16 KiB: N <= 65536
constexpr size_t kNoAllocBytes = kNoAllocTileFloats * sizeof(float) + (size_t)kNoAllocCounters * sizeof(int);

static __device__ __align__(256) unsigned char scratch[kNoAllocBytes];

constexpr int kMaxDevices = 64;
unsigned char* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each GPU set up so far

__global__ void noalloc_clear_kernel(int* counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
}

}  // namespace

int noalloc_setup(int device_index) {
  if (device_index < 0 || device_index >= kMaxDevices)
    return set_error(TLHIP_ERR_INVALID, "noalloc: device index %d out of range", device_index);
  if (g_scratch_ptr[device_index]) return TLHIP_OK;
  // the current device is `device_index` (tlhip_init has just selected it)
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess || !ptr)
    return set_error(TLHIP_ERR_DEVICE, "noalloc: hipGetSymbolAddress(scratch) failed: %s", hipGetErrorString(e));
  g_scratch_ptr[device_index] = (unsigned char*)ptr;
  return TLHIP_OK;
}

}  // namespace tlhip

using namespace tlhip;

extern "C" int tlhip_gemv_noalloc(const tlhip_qweight_t* w, const void* x, int x_dtype, int64_t m, void* y, int y_dtype,
                                  float alpha, const tlhip_epilogue_t* epilogue, tlhip_stream_t stream) {
  TLHIP_REQUIRE_INIT();
  Problem p;
  int rc = make_problem(w, x, x_dtype, m, y, y_dtype, alpha, epilogue, &p, "gemv_noalloc");
  if (rc) return rc;
  if (m > 16) return set_error(TLHIP_ERR_INVALID, "gemv_noalloc: M=%lld above 16", (long long)m);
  if (p.m == 0 || p.n == 0) return TLHIP_OK;
  int dev = -1;
  TLHIP_CHECK_HIP(hipGetDevice(&dev));
  // the array's address differs from GPU to GPU: the one of the library's device is only
  // right while that device is the calling thread's current one (as every launch needs)
  if (dev != device_index())
    return set_error(TLHIP_ERR_STATE, "gemv_noalloc: device %d is current, the library was initialised on device %d",
                     dev, device_index());
  if (dev < 0 || dev >= kMaxDevices || !g_scratch_ptr[dev])
    return set_error(TLHIP_ERR_STATE, "gemv_noalloc: the scratch of device %d was not set up by tlhip_init", dev);
  // the configuration and the route (one launch, or the rows in chunks) tlhip_gemv would
  // take for this problem, selected exactly as it selects them; every launch of the route
  // combines its K slices through the fixed array, one launch after the other
  const int ks = gemv_route_k_slices(p);
  hipStream_t s = resolve_stream(stream);
  SplitScratch sc;
  sc.tiles = (float*)g_scratch_ptr[dev];
  sc.counters = (int*)(g_scratch_ptr[dev] + kNoAllocTileFloats * sizeof(float));
  sc.tile_floats = kNoAllocTileFloats;
  sc.ncounters = kNoAllocCounters;
  if (ks > 1) {
    const int64_t nblocks = (p.n + 15) / 16;
    const size_t need = (size_t)nblocks * ks * 256;
    if (need > kNoAllocTileFloats || nblocks > kNoAllocCounters)
      return set_error(TLHIP_ERR_INVALID,
                       "gemv_noalloc: N=%lld with %d K slices needs %zu bytes of partial tiles and %lld counters; the "
                       "fixed scratch holds %zu bytes and %d counters (use tlhip_gemv)",
                       (long long)p.n, ks, need * sizeof(float), (long long)nblocks, kNoAllocTileFloats * sizeof(float),
                       kNoAllocCounters);
    // what must start at zero: the arrival counters of this launch's row blocks (a fill
    // kernel, not a memset node: the call may be under graph capture)
    hipLaunchKernelGGL(noalloc_clear_kernel, dim3((unsigned)((nblocks + 255) / 256)), dim3(256), 0, s, sc.counters,
                       (int)nblocks);
    TLHIP_CHECK_HIP(hipGetLastError());
  }
  p.scratch = &sc;
  return run_gemv_route(p, s);
}
