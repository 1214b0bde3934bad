// placeholder until the MFMA prefill kernel lands
#include "device_utils.h"
namespace tlhip {
bool gemm_config_applicable(const Problem&, const tlhip_kernel_config_t&, const char** why) {
  if (why) *why = "prefill GEMM not built";
  return false;
}
int launch_gemm(const Problem&, const tlhip_kernel_config_t&, hipStream_t) {
  return set_error(TLHIP_ERR_INVALID, "prefill GEMM not built");
}
}  // namespace tlhip
