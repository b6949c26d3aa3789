// Decode kernel instantiations with the gated-MLP epilogue (act(x @ gate) * (x @ up)), kept in
// their own translation unit so that they compile in parallel with the plain ones.  The
// launcher offers them for one and two activation rows only (grouped launches: tokens).
#include "q4_gemv_kernels.cuh"

namespace q4host {

using q4::GemvParams;

template <int DTYPE, int RMAX, bool MOE>
static void launch_fused(const GemvParams& gp, bool static128, dim3 grid, dim3 block, size_t smem,
                         hipStream_t stream) {
  using namespace q4;
  if (static128) {
    auto k = gemv_gptq_kernel<DTYPE, RMAX, 4, true, 8, true, MOE>;
    if (smem > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, block, smem, stream, gp);
  } else {
    auto k = gemv_gptq_kernel<DTYPE, RMAX, 4, false, 8, true, MOE>;
    if (smem > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, block, smem, stream, gp);
  }
}

template <bool MOE>
static void launch_fused_any(const GemvParams& gp, int dtype, int rmax, bool static128, dim3 grid, dim3 block,
                             size_t smem, hipStream_t stream) {
  if (dtype == Q4_DTYPE_F16) {
    if (rmax == 1) launch_fused<Q4_DTYPE_F16, 1, MOE>(gp, static128, grid, block, smem, stream);
    else launch_fused<Q4_DTYPE_F16, 2, MOE>(gp, static128, grid, block, smem, stream);
  } else {
    if (rmax == 1) launch_fused<Q4_DTYPE_BF16, 1, MOE>(gp, static128, grid, block, smem, stream);
    else launch_fused<Q4_DTYPE_BF16, 2, MOE>(gp, static128, grid, block, smem, stream);
  }
}

// grouped: the mixture-of-experts variants (blockIdx.z is the expert)
void launch_gemv_gate_up(const GemvParams& gp, int dtype, int rmax, bool static128, dim3 grid, dim3 block,
                         size_t smem, hipStream_t stream, bool grouped) {
  if (grouped) launch_fused_any<true>(gp, dtype, rmax, static128, grid, block, smem, stream);
  else launch_fused_any<false>(gp, dtype, rmax, static128, grid, block, smem, stream);
}

}  // namespace q4host
