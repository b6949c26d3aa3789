// Instantiations of the instruction-lean contiguous-group decode kernel (q4_gemv_lean.cuh), in
// their own translation unit so that they compile in parallel with the other decode kernels.
#include "q4_gemv_lean.cuh"

namespace q4host {

using q4::GemvParams;

template <int DTYPE, int MP, int PF = 2>
static void launch_one(const GemvParams& gp, dim3 grid, dim3 block, size_t smem, hipStream_t stream) {
  auto k = q4::gemv_gptq_lean_kernel<DTYPE, MP, PF>;
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, block, smem, stream, gp);
}

template <int DTYPE>
static void launch_dtype(const GemvParams& gp, int mp, dim3 grid, dim3 block, size_t smem, hipStream_t stream) {
  switch (mp) {
    case 1: launch_one<DTYPE, 1>(gp, grid, block, smem, stream); break;
    case 2: launch_one<DTYPE, 2>(gp, grid, block, smem, stream); break;
    case 4: launch_one<DTYPE, 4>(gp, grid, block, smem, stream); break;
    case 8: launch_one<DTYPE, 8>(gp, grid, block, smem, stream); break;
    default: launch_one<DTYPE, 16>(gp, grid, block, smem, stream); break;
  }
}

// mp: activation rows of a workgroup padded to a power of two (1, 2, 4, 8, 16)
void launch_gemv_lean(const GemvParams& gp, int dtype, int mp, dim3 grid, dim3 block, size_t smem,
                      hipStream_t stream) {
  if (dtype == Q4_DTYPE_F16) launch_dtype<Q4_DTYPE_F16>(gp, mp, grid, block, smem, stream);
  else launch_dtype<Q4_DTYPE_BF16>(gp, mp, grid, block, smem, stream);
}

}  // namespace q4host
