// Act-order without per-weight lookups: the rows of a GPTQ matrix are put into group order
// once at load time and the activation columns follow the same order at run time, after which
// the contiguous-group kernels apply.  The reference's exllamav2 path does the same
// (QMatrix::make_sequential + make_sequential_kernel, cuda/q_matrix.cu:524-640, and the
// b_q_perm gather of the activations in its GEMM, cuda/q_gemm_kernel_gptq.cuh:116).
#include "q4_common.cuh"

namespace q4 {

// out word (r, n) = nibbles of source rows perm[8r .. 8r+7] of column n.  One thread per
// column and packed row: the eight source words are coalesced along n.
__global__ __launch_bounds__(256) void make_sequential_kernel(const uint32_t* __restrict__ qweight,
                                                              const int32_t* __restrict__ perm,
                                                              uint32_t* __restrict__ out, int K, int N) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int r = blockIdx.y;
  if (n >= N) return;
  uint32_t word = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int src = min(max(perm[8 * r + i], 0), K - 1);  // a bad index reads a wrong row, never outside
    const uint32_t w = qweight[(size_t)(src >> 3) * N + n];
    word |= ((w >> ((src & 7) * 4)) & 0xFu) << (4 * i);
  }
  out[(size_t)r * N + n] = word;
}

// out[m][i] = x[m][perm[i]] for 16-bit elements.  A thread gathers eight neighbours of the output
// row (one 16-byte store); the reads hit a row of x that stays in L2.
__global__ __launch_bounds__(256) void gather_columns_kernel(const uint16_t* __restrict__ x,
                                                             const int32_t* __restrict__ perm,
                                                             uint16_t* __restrict__ out, int M, int K) {
  const int vec_per_row = K >> 3;
  const long total = (long)M * vec_per_row;
  for (long v = (long)blockIdx.x * blockDim.x + threadIdx.x; v < total; v += (long)gridDim.x * blockDim.x) {
    const long m = v / vec_per_row;
    const int c = (int)(v - m * vec_per_row) * 8;
    const uint16_t* row = x + (size_t)m * K;
    const uint4_t p0 = *(const uint4_t*)(perm + c);
    const uint4_t p1 = *(const uint4_t*)(perm + c + 4);
    const uint32_t idx[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
    uint32_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = row[min(max((int)idx[i], 0), K - 1)];
    uint4_t o;
    o.x = h[0] | (h[1] << 16);
    o.y = h[2] | (h[3] << 16);
    o.z = h[4] | (h[5] << 16);
    o.w = h[6] | (h[7] << 16);
    *(uint4_t*)(out + (size_t)m * K + c) = o;
  }
}

// Grouped form: sorted row r of expert e (offsets[e] <= r < offsets[e + 1]) becomes
// x[x_rows ? x_rows[r] : r][perms[e][.]].  Output [pairs, K] in sorted order.
__global__ __launch_bounds__(256) void moe_gather_columns_kernel(const uint16_t* __restrict__ x,
                                                                 const int32_t* __restrict__ x_rows,
                                                                 const int32_t* __restrict__ offsets,
                                                                 const int32_t* __restrict__ perms,
                                                                 uint16_t* __restrict__ out, int num_experts,
                                                                 int pairs, int K) {
  const int vec_per_row = K >> 3;
  const long total = (long)pairs * vec_per_row;
  for (long v = (long)blockIdx.x * blockDim.x + threadIdx.x; v < total; v += (long)gridDim.x * blockDim.x) {
    const int r = (int)(v / vec_per_row);
    const int c = (int)(v - (long)r * vec_per_row) * 8;
    int lo = 0, hi = num_experts;  // expert of row r: the last e with offsets[e] <= r
    while (hi - lo > 1) {
      const int mid = (lo + hi) >> 1;
      if (offsets[mid] <= r) lo = mid; else hi = mid;
    }
    const uint16_t* row = x + (size_t)(x_rows != nullptr ? x_rows[r] : r) * K;
    const int32_t* perm = perms + (size_t)lo * K;
    const uint4_t p0 = *(const uint4_t*)(perm + c);
    const uint4_t p1 = *(const uint4_t*)(perm + c + 4);
    const uint32_t idx[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
    uint32_t h[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = row[min(max((int)idx[i], 0), K - 1)];
    uint4_t o;
    o.x = h[0] | (h[1] << 16);
    o.y = h[2] | (h[3] << 16);
    o.z = h[4] | (h[5] << 16);
    o.w = h[6] | (h[7] << 16);
    *(uint4_t*)(out + (size_t)r * K + c) = o;
  }
}

// Many rows: a workgroup stages one row of x in LDS with 16-byte loads and gathers from there,
// so that global memory sees only coalesced traffic (the direct kernels above read 2-byte
// elements scattered over the row).  perms == one permutation when offsets is nullptr.
__global__ __launch_bounds__(256) void gather_rows_lds_kernel(const uint16_t* __restrict__ x,
                                                              const int32_t* __restrict__ x_rows,
                                                              const int32_t* __restrict__ offsets,
                                                              const int32_t* __restrict__ perms,
                                                              uint16_t* __restrict__ out, int num_experts, int rows,
                                                              int K) {
  extern __shared__ __align__(16) uint16_t row_lds[];  // [K]
  const int vec_per_row = K >> 3;
  for (int r = blockIdx.x; r < rows; r += gridDim.x) {
    const int32_t* perm = perms;
    if (offsets != nullptr) {
      int lo = 0, hi = num_experts;
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (offsets[mid] <= r) lo = mid; else hi = mid;
      }
      perm += (size_t)lo * K;
    }
    const uint16_t* src = x + (size_t)(x_rows != nullptr ? x_rows[r] : r) * K;
    for (int v = threadIdx.x; v < vec_per_row; v += 256) ((uint4_t*)row_lds)[v] = ((const uint4_t*)src)[v];
    __syncthreads();
    for (int v = threadIdx.x; v < vec_per_row; v += 256) {
      const uint4_t p0 = *(const uint4_t*)(perm + v * 8);
      const uint4_t p1 = *(const uint4_t*)(perm + v * 8 + 4);
      const uint32_t idx[8] = {p0.x, p0.y, p0.z, p0.w, p1.x, p1.y, p1.z, p1.w};
      uint32_t h[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) h[i] = row_lds[min(max((int)idx[i], 0), K - 1)];
      uint4_t o;
      o.x = h[0] | (h[1] << 16);
      o.y = h[2] | (h[3] << 16);
      o.z = h[4] | (h[5] << 16);
      o.w = h[6] | (h[7] << 16);
      ((uint4_t*)(out + (size_t)r * K))[v] = o;
    }
    __syncthreads();
  }
}

}  // namespace q4

namespace q4host {

// rows from which the LDS-staged kernel is used (fewer rows leave most CUs without a workgroup)
static constexpr int kGatherLdsRows = 128;

static bool launch_gather_lds(const void* x, const int32_t* x_rows, const int32_t* offsets, const int32_t* perms,
                              void* out, int num_experts, int rows, int K, hipStream_t stream) {
  const size_t smem = (size_t)K * 2;
  if (rows < kGatherLdsRows || smem > 64 * 1024) return false;
  const int blocks = rows < 2048 ? rows : 2048;
  hipLaunchKernelGGL(q4::gather_rows_lds_kernel, dim3((unsigned)blocks), dim3(256), smem, stream, (const uint16_t*)x,
                     x_rows, offsets, perms, (uint16_t*)out, num_experts, rows, K);
  return true;
}


int launch_moe_gather_columns(const void* x, const int32_t* x_rows, const int32_t* offsets, const int32_t* perms,
                              void* out, int num_experts, int pairs, int K, hipStream_t stream) {
  const long total = (long)pairs * (K / 8);
  long blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  if (blocks < 1) blocks = 1;
  if (!launch_gather_lds(x, x_rows, offsets, perms, out, num_experts, pairs, K, stream)) {
    hipLaunchKernelGGL(q4::moe_gather_columns_kernel, dim3((unsigned)blocks), dim3(256), 0, stream,
                       (const uint16_t*)x, x_rows, offsets, perms, (uint16_t*)out, num_experts, pairs, K);
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_moe_gather_columns: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}


int launch_make_sequential(const uint32_t* qweight, const int32_t* perm, uint32_t* out, int K, int N,
                           hipStream_t stream) {
  dim3 grid((unsigned)((N + 255) / 256), (unsigned)(K / 8));
  hipLaunchKernelGGL(q4::make_sequential_kernel, grid, dim3(256), 0, stream, qweight, perm, out, K, N);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_gptq_make_sequential: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

int launch_gather_columns(const void* x, const int32_t* perm, void* out, int M, int K, hipStream_t stream) {
  const long total = (long)M * (K / 8);
  long blocks = (total + 255) / 256;
  if (blocks > 8192) blocks = 8192;
  if (blocks < 1) blocks = 1;
  if (!launch_gather_lds(x, nullptr, nullptr, perm, out, 1, M, K, stream)) {
    hipLaunchKernelGGL(q4::gather_columns_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (const uint16_t*)x,
                       perm, (uint16_t*)out, M, K);
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_gather_columns: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
