// The instances of the skinny matrix-core GEMV for 17..64 activation rows: two or four
// tiles of 16 rows per weight row block (gemv_mfma_kernel.h), single problem, at most 8
// waves per workgroup.  A translation unit of their own, compiled beside the others.
#include "gemv_mfma_kernel.h"

namespace tlhip {

int launch_mfma_rows(int tiles, int format, int group_size, int64_t k, int unroll, int line, const MfmaArgs& a, int grid,
                     int threads, size_t lds_bytes, hipStream_t stream) {
  if (tiles == 2) return launch_mfma_instance<false, 2>(format, group_size, k, unroll, line, a, grid, threads, lds_bytes, stream);
  if (tiles == 4) return launch_mfma_instance<false, 4>(format, group_size, k, unroll, line, a, grid, threads, lds_bytes, stream);
  return set_error(TLHIP_ERR_INVALID, "gemv_mfma: %d tiles of activation rows (2 or 4)", tiles);
}

int prepare_mfma_rows() {
  const int rc = prepare_mfma_instances<false, 2>();
  return rc ? rc : prepare_mfma_instances<false, 4>();
}

}  // namespace tlhip
