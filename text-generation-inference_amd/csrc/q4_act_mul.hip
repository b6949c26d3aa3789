// Unfused tail of a gated MLP: y[M, I] = act(gate_up[:, :I]) * gate_up[:, I:], for the
// weights whose linear kernels have no fused epilogue (AWQ layout, act-order).  HBM-bound
// elementwise pass: 16-byte loads of both halves, one 16-byte store.
#include "q4_common.cuh"

namespace q4 {

template <int DTYPE>
__global__ __launch_bounds__(256) void act_mul_kernel(const uint16_t* __restrict__ gate_up,
                                                      uint16_t* __restrict__ y, int M, int inter, int act) {
  const int vec_per_row = inter >> 3;  // 8 values per 16-byte vector
  const long total = (long)M * vec_per_row;
  for (long v = (long)blockIdx.x * blockDim.x + threadIdx.x; v < total; v += (long)gridDim.x * blockDim.x) {
    const long m = v / vec_per_row;
    const int c = (int)(v - m * vec_per_row) * 8;
    const uint16_t* row = gate_up + (size_t)m * 2 * inter;
    const uint4_t g = *(const uint4_t*)(row + c);
    const uint4_t u = *(const uint4_t*)(row + inter + c);
    const uint32_t gw[4] = {g.x, g.y, g.z, g.w};
    const uint32_t uw[4] = {u.x, u.y, u.z, u.w};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const uint32_t lo = act_mul<DTYPE>((uint16_t)(gw[i] & 0xFFFFu), (uint16_t)(uw[i] & 0xFFFFu), act);
      const uint32_t hi = act_mul<DTYPE>((uint16_t)(gw[i] >> 16), (uint16_t)(uw[i] >> 16), act);
      o[i] = lo | (hi << 16);
    }
    *(uint4_t*)(y + (size_t)m * inter + c) = uint4_t{o[0], o[1], o[2], o[3]};
  }
}

}  // namespace q4

namespace q4host {

int launch_act_mul(const void* gate_up, void* y, int M, int inter, int dtype, int act, hipStream_t stream) {
  if (inter % 8 != 0) {
    set_error("q4_act_mul: the intermediate size %d must be a multiple of 8", inter);
    return Q4_ERR_UNSUPPORTED;
  }
  const long total = (long)M * (inter / 8);
  long blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;  // grid-stride beyond 32 workgroups per CU
  if (blocks < 1) blocks = 1;
  if (dtype == Q4_DTYPE_F16)
    hipLaunchKernelGGL(q4::act_mul_kernel<Q4_DTYPE_F16>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const uint16_t*)gate_up, (uint16_t*)y, M, inter, act);
  else
    hipLaunchKernelGGL(q4::act_mul_kernel<Q4_DTYPE_BF16>, dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const uint16_t*)gate_up, (uint16_t*)y, M, inter, act);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_act_mul: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
