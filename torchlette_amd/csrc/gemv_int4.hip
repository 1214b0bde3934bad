// VALU decode GEMV kernels for one weight format (see gemv_kernel.h).
#include "gemv_kernel.h"

namespace tlhip {
TLHIP_DEFINE_GEMV_FORMAT(int4, TLHIP_FMT_INT4_GROUPED)
}  // namespace tlhip
