// Dense dequantization W[K, N] = round_once(s * (q - z)) for both checkpoint layouts.
//
// HBM-bound on the 2-byte-per-weight store side (0.5 B read + 2 B written per weight),
// so the kernel is organised around wide coalesced stores: a GPTQ thread owns a
// 4-column x 8-row patch (one 128-bit load, eight 64-bit stores that are contiguous
// across the wavefront); an AWQ thread owns one word = 8 adjacent columns of one row
// (one 128-bit store).  The arithmetic is the scalar dequant_one() so the result is the
// reference's value bit for bit, including act-order group lookup through g_idx.
#include "q4_common.cuh"

namespace q4 {

template <int DTYPE>
__global__ __launch_bounds__(256) void dequant_gptq_kernel(
    const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
    const half_t* __restrict__ scales, const int32_t* __restrict__ g_idx,
    uint16_t* __restrict__ w_out, int K, int N, int groupsize, int num_groups) {
  const int n4 = blockIdx.x * blockDim.x + threadIdx.x;  // group of 4 columns
  const int n = n4 * 4;
  if (n >= N) return;
  for (int r = blockIdx.y; r < K / 8; r += gridDim.y) {  // packed row (8 K rows)
  const uint4_t words = *(const uint4_t*)(qweight + (size_t)r * N + n);
  const uint32_t w[4] = {words.x, words.y, words.z, words.w};
  const int zshift = (n & 7) * 4;
  int g_prev = -1;
  uint32_t zbits = 0;
  half_t s[4] = {};
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const int k = r * 8 + j;
    int g = g_idx ? g_idx[k] : k / groupsize;
    g = min(max(g, 0), num_groups - 1);
    if (g != g_prev) {
      g_prev = g;
      zbits = gptq_zero_plus_one(qzeros[(size_t)g * (N / 8) + (n >> 3)]) >> zshift;
      const uint2_t sraw = *(const uint2_t*)(scales + (size_t)g * N + n);
      // as_half2() takes the element by value: a bit cast applied directly to a vector
      // element expression reads element 0 with this compiler.
      const half2_t s01 = as_half2(sraw.x), s23 = as_half2(sraw.y);
      s[0] = s01.x;
      s[1] = s01.y;
      s[2] = s23.x;
      s[3] = s23.y;
    }
    uint16_t o[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const int q = (w[t] >> (4 * j)) & 0xF;
      const int z = (zbits >> (4 * t)) & 0xF;
      o[t] = dequant_one<DTYPE>(s[t], q, z);
    }
    uint2_t packed;
    packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
    packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
    *(uint2_t*)(w_out + (size_t)k * N + n) = packed;
  }
  }
}

template <int DTYPE>
__global__ __launch_bounds__(256) void dequant_awq_kernel(
    const uint32_t* __restrict__ qweight, const uint32_t* __restrict__ qzeros,
    const half_t* __restrict__ scales, uint16_t* __restrict__ w_out, int K, int N, int groupsize,
    int num_groups) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;  // packed column (8 N columns)
  const int NC = N / 8;
  if (c >= NC) return;
  for (int k = blockIdx.y; k < K; k += gridDim.y) {
  const int g = min(k / groupsize, num_groups - 1);
  const uint32_t w = qweight[(size_t)k * NC + c];
  const uint32_t z = qzeros[(size_t)g * NC + c];
  const uint4_t sraw = *(const uint4_t*)(scales + (size_t)g * N + c * 8);
  const uint32_t su[4] = {sraw.x, sraw.y, sraw.z, sraw.w};
  uint16_t o[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {  // logical column 8c + i lives at nibble awq_position(i)
    const int p = awq_position(i);
    const int q = (w >> (4 * p)) & 0xF;
    const int zz = (z >> (4 * p)) & 0xF;
    const half2_t sp = as_half2(su[i >> 1]);
    o[i] = dequant_one<DTYPE>((i & 1) ? sp.y : sp.x, q, zz);
  }
  uint4_t packed;
  packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
  packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
  packed.z = (uint32_t)o[4] | ((uint32_t)o[5] << 16);
  packed.w = (uint32_t)o[6] | ((uint32_t)o[7] << 16);
  *(uint4_t*)(w_out + (size_t)k * N + c * 8) = packed;
  }
}

}  // namespace q4

namespace q4host {

int launch_dequant(const q4_weight* w, void* w_out, int dtype, hipStream_t stream) {
  using namespace q4;
  const int K = w->K, N = w->N;
  if (K == 0 || N == 0) return Q4_OK;
  if (w->layout == Q4_LAYOUT_GPTQ) {
    dim3 block(256);
    dim3 grid((N / 4 + 255) / 256, K / 8 < 32768 ? K / 8 : 32768);
    if (dtype == Q4_DTYPE_F16) {
      hipLaunchKernelGGL(dequant_gptq_kernel<Q4_DTYPE_F16>, grid, block, 0, stream, w->qweight,
                         w->qzeros, (const half_t*)w->scales, w->g_idx, (uint16_t*)w_out, K, N,
                         w->groupsize, w->num_groups);
    } else {
      hipLaunchKernelGGL(dequant_gptq_kernel<Q4_DTYPE_BF16>, grid, block, 0, stream, w->qweight,
                         w->qzeros, (const half_t*)w->scales, w->g_idx, (uint16_t*)w_out, K, N,
                         w->groupsize, w->num_groups);
    }
  } else {
    dim3 block(256);
    dim3 grid((N / 8 + 255) / 256, K < 32768 ? K : 32768);
    if (dtype == Q4_DTYPE_F16) {
      hipLaunchKernelGGL(dequant_awq_kernel<Q4_DTYPE_F16>, grid, block, 0, stream, w->qweight,
                         w->qzeros, (const half_t*)w->scales, (uint16_t*)w_out, K, N, w->groupsize,
                         w->num_groups);
    } else {
      hipLaunchKernelGGL(dequant_awq_kernel<Q4_DTYPE_BF16>, grid, block, 0, stream, w->qweight,
                         w->qzeros, (const half_t*)w->scales, (uint16_t*)w_out, K, N, w->groupsize,
                         w->num_groups);
    }
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_dequant: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
