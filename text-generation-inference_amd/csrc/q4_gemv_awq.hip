// Instantiations and launcher of the AWQ-layout decode kernel (q4_gemv_awq.cuh).
#include "q4_gemv_awq.cuh"

namespace q4host {

template <typename Kernel>
static void launch_one(Kernel k, const q4::GemvParams& gp, dim3 grid, dim3 block, size_t smem, hipStream_t stream) {
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, block, smem, stream, gp);
}

template <int DTYPE>
static void launch_dtype(const q4::GemvParams& gp, int row_groups, dim3 grid, dim3 block, size_t smem, hipStream_t stream) {
  using namespace q4;
  if (row_groups <= 1) launch_one(gemv_awq_diag_kernel<DTYPE, 1>, gp, grid, block, smem, stream);
  else launch_one(gemv_awq_diag_kernel<DTYPE, 2>, gp, grid, block, smem, stream);
}

void launch_gemv_awq_diag(const q4::GemvParams& gp, int dtype, int row_groups, dim3 grid, dim3 block, size_t smem,
                          hipStream_t stream) {
  if (dtype == Q4_DTYPE_F16) launch_dtype<Q4_DTYPE_F16>(gp, row_groups, grid, block, smem, stream);
  else launch_dtype<Q4_DTYPE_BF16>(gp, row_groups, grid, block, smem, stream);
}

}  // namespace q4host
