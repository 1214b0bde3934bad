// The skinny matrix-core GEMV's kernel instances with a problem table (several Linears
// that share their activations in one launch): see gemv_mfma_kernel.h.
#include "gemv_mfma_kernel.h"

namespace tlhip {

int launch_mfma_grouped(int format, int group_size, int64_t k, int unroll, int line, const MfmaArgs& a, int grid, int threads,
                        size_t lds_bytes, hipStream_t stream) {
  return launch_mfma_instance<true>(format, group_size, k, unroll, line, a, grid, threads, lds_bytes, stream);
}
int prepare_mfma_grouped() { return prepare_mfma_instances<true>(); }

}  // namespace tlhip
