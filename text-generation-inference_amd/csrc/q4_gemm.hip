// Prefill path placeholder translation unit: filled in by the MFMA GEMM kernel.
#include "q4_common.cuh"

namespace q4host {
bool gemm_supported(const q4_weight*, int, int) { return false; }
int launch_gemm(const q4_weight*, const void*, const void*, void*, int, int, hipStream_t) {
  set_error("q4_linear(gemm): not built");
  return Q4_ERR_UNSUPPORTED;
}
}  // namespace q4host
