// The 4x4x4 matrix-core form of the decode GEMV (int4 grouped weights, f16 activations,
// up to four activation rows): see gemv_kernel.h.
#include "gemv_kernel.h"

namespace tlhip {

int launch_gemv_mf4_int4(int u, const GemvArgs& a, int threads, int grid, size_t lds_bytes, hipStream_t stream) {
  switch (u) {
    case 2: return launch_t<TLHIP_FMT_INT4_GROUPED, _Float16, 4, 1, 2, true>(a, threads, grid, lds_bytes, stream);
    case 4: return launch_t<TLHIP_FMT_INT4_GROUPED, _Float16, 4, 1, 4, true>(a, threads, grid, lds_bytes, stream);
    case 8: return launch_t<TLHIP_FMT_INT4_GROUPED, _Float16, 4, 1, 8, true>(a, threads, grid, lds_bytes, stream);
  }
  return set_error(TLHIP_ERR_INVALID, "gemv: chunks in flight = %d is not built for the 4x4x4 form", u);
}

}  // namespace tlhip
