// A read-only streaming kernel used as the measuring stick for the decode
// GEMV: it does what the GEMV must do at the very least (fetch every byte of
// the packed weight once with 16-byte loads) and nothing else.  Timed with the
// same back-to-back launches as the GEMV, it shows how much of the 8 TB/s peak a
// single launch of a given size can reach at all once launch overhead and the
// ramp of the memory pipeline are paid.
//
// A benchmark instrument, not part of the product: built into its own shared
// object (libtlhip_bench.so), which only the benchmark loads.
#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void hbm_read_probe_kernel(const u32x4* __restrict__ p, size_t n16,
                                                            uint32_t* __restrict__ sink) {
  const size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  uint32_t acc = 0;
  for (size_t i = tid; i < n16; i += stride) {
    const u32x4 v = __builtin_nontemporal_load(p + i);
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;  // keeps the loads alive; practically never taken
}

}  // namespace

// Reads `bytes` bytes at `ptr` (device, 16-byte aligned) once on `stream` (a hipStream_t;
// null = the default stream) and discards them; `sink4` is 4 writable device bytes.
// Returns 0, -1 for bad arguments, or the HIP error code of the launch.
extern "C" int tlbench_hbm_read_probe(const void* ptr, size_t bytes, void* sink4, void* stream) {
  if (!ptr || !sink4 || ((uintptr_t)ptr & 15) != 0) return -1;
  const size_t n16 = bytes / 16;
  if (n16 == 0) return 0;
  int dev = 0, cus = 0;
  if (hipGetDevice(&dev) != hipSuccess) return -1;
  if (hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0) return -1;
  const size_t blocks = (n16 + 255) / 256;
  const size_t cap = (size_t)cus * 8;  // 8 workgroups of 4 waves per CU: the best measured shape
  const int grid = (int)(blocks < cap ? blocks : cap);
  hipLaunchKernelGGL(hbm_read_probe_kernel, dim3(grid), dim3(256), 0, (hipStream_t)stream, (const u32x4*)ptr, n16,
                     (uint32_t*)sink4);
  return (int)hipGetLastError();
}
