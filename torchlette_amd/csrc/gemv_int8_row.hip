// VALU decode GEMV kernels for one weight format (see gemv_kernel.h).
#include "gemv_kernel.h"

namespace tlhip {
TLHIP_DEFINE_GEMV_FORMAT(int8_row, TLHIP_FMT_INT8_ROW)
}  // namespace tlhip
