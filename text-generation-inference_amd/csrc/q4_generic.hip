// Shape-agnostic fallback: y = x @ dequant(W) for any K % 8 == 0, N % 8 == 0, any M, both
// layouts, with or without g_idx, any groupsize.  One thread per output column, four
// activation rows per pass, fp32 accumulation in K order.  It exists so that every shape
// the reference accepts has a HIP path; the decode and prefill kernels cover the aligned
// shapes real checkpoints have.
#include "q4_common.cuh"

namespace q4 {

constexpr int kGenericRows = 4;

template <int DTYPE, int LAYOUT>
__global__ __launch_bounds__(256) void generic_kernel(Problem p) {
  const int n = blockIdx.x * blockDim.x + threadIdx.x;
  const int m0 = blockIdx.y * kGenericRows;
  if (n >= p.N) return;
  const int NC = p.N / 8;
  float acc[kGenericRows] = {};
  int g_prev = -1;
  half_t s = (half_t)0.0f;
  int z = 0;
  const int shift_n = (LAYOUT == Q4_LAYOUT_AWQ) ? 4 * awq_position(n & 7) : 4 * (n & 7);
  for (int k8 = 0; k8 < p.K; k8 += 8) {
    uint32_t wword = 0;
    if constexpr (LAYOUT == Q4_LAYOUT_GPTQ) wword = p.qweight[(size_t)(k8 >> 3) * p.N + n];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int k = k8 + j;
      int g = p.g_idx ? p.g_idx[k] : k / p.groupsize;
      g = min(max(g, 0), p.num_groups - 1);
      if (g != g_prev) {
        g_prev = g;
        s = p.scales[(size_t)g * p.N + n];
        uint32_t zw = p.qzeros[(size_t)g * NC + (n >> 3)];
        if constexpr (LAYOUT == Q4_LAYOUT_GPTQ) zw = gptq_zero_plus_one(zw);
        z = (zw >> shift_n) & 0xF;
      }
      int q;
      if constexpr (LAYOUT == Q4_LAYOUT_GPTQ) {
        q = (wword >> (4 * j)) & 0xF;
      } else {
        q = (p.qweight[(size_t)k * NC + (n >> 3)] >> shift_n) & 0xF;
      }
      const uint16_t wb = dequant_one<DTYPE>(s, q, z);
      float wf;
      if constexpr (DTYPE == Q4_DTYPE_F16) {
        wf = (float)__builtin_bit_cast(half_t, wb);
      } else {
        wf = bf16_bits_to_f32(wb);
      }
#pragma unroll
      for (int r = 0; r < kGenericRows; ++r) {
        if (m0 + r < p.M) acc[r] = fmaf(load_act<DTYPE>(p.x, (size_t)(m0 + r) * p.K + k), wf, acc[r]);
      }
    }
  }
#pragma unroll
  for (int r = 0; r < kGenericRows; ++r) {
    if (m0 + r < p.M) {
      ((uint16_t*)p.y)[(size_t)(m0 + r) * p.N + n] = finish_output<DTYPE>(acc[r], p.bias, n);
    }
  }
}

}  // namespace q4

namespace q4host {

int launch_generic(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                   hipStream_t stream) {
  using namespace q4;
  if (M == 0 || w->N == 0) return Q4_OK;
  Problem p{w->qweight, w->qzeros, (const half_t*)w->scales, w->g_idx, x, bias, y,
            M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  dim3 block(256);
  const unsigned gy = (unsigned)((M + kGenericRows - 1) / kGenericRows);
  if (gy > 65535u) {
    set_error("q4_linear(generic): M=%d too large", M);
    return Q4_ERR_UNSUPPORTED;
  }
  dim3 grid((w->N + 255) / 256, gy);
  const bool awq = w->layout == Q4_LAYOUT_AWQ;
  if (dtype == Q4_DTYPE_F16) {
    if (awq) hipLaunchKernelGGL((generic_kernel<Q4_DTYPE_F16, Q4_LAYOUT_AWQ>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((generic_kernel<Q4_DTYPE_F16, Q4_LAYOUT_GPTQ>), grid, block, 0, stream, p);
  } else {
    if (awq) hipLaunchKernelGGL((generic_kernel<Q4_DTYPE_BF16, Q4_LAYOUT_AWQ>), grid, block, 0, stream, p);
    else hipLaunchKernelGGL((generic_kernel<Q4_DTYPE_BF16, Q4_LAYOUT_GPTQ>), grid, block, 0, stream, p);
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(generic): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
