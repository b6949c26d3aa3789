// The inner loop of the GPTQ solver (the reference's GPTQ.fasterquant,
// server/text_generation_server/layers/gptq/quantize.py:294-331): inside a block of up to 128
// input columns every column is quantized in turn and its error is fed forward into the columns
// not yet quantized, through the rows of the upper Cholesky factor U of the inverse Hessian.
// Output rows are independent: one wave owns one row and keeps the block's 128 weights in
// registers (two per lane), so the 128 dependent steps cost a broadcast, a handful of VALU
// operations and one LDS row read each instead of several kernel launches.  The block of U
// sits in LDS, shared by the sixteen waves of a workgroup (the loop is a chain of dependent
// operations: many resident waves per CU hide its latency).  The update of the columns behind the
// block (W[:, i2:] -= Err @ U[i1:i2, i2:]) is a plain GEMM and stays with the caller.
#include "q4_common.cuh"

namespace q4 {

constexpr int kSolveBlock = 128;  // columns per block (two per lane)
constexpr int kSolveWaves = 16;   // rows (waves) per workgroup: they share the LDS copy of the block of U

struct SolveParams {
  float* __restrict__ W;          // [rows, K] row-major, current weights; block columns are read
  const float* __restrict__ U;    // [K, K] row-major, upper triangular: inv(H) = U^T U
  float* __restrict__ Q;          // [rows, K] quantized (dequantized values) of the block's columns
  float* __restrict__ Err;        // [rows, kSolveBlock] errors (w - q) / U_ii of the block's columns
  float* __restrict__ loss;       // [rows] += sum of (w - q)^2 / U_ii^2 / 2
  float* __restrict__ scale;      // [rows, G]
  float* __restrict__ zero;       // [rows, G]
  int rows, K, i1, count;
  int groupsize;                  // <= 0: one set of parameters per row, already in scale / zero
  int G, sym;
  int given;                      // groups starting in the block: parameters already in scale / zero
};

__device__ __forceinline__ float wave_min(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fminf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

__global__ __launch_bounds__(64 * kSolveWaves) void gptq_solve_block_kernel(SolveParams sp) {
  extern __shared__ __align__(16) float u_lds[];  // [count][kSolveBlock]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int count = sp.count, K = sp.K;
  for (int idx = tid; idx < count * kSolveBlock; idx += 64 * kSolveWaves) {
    const int r = idx / kSolveBlock, c = idx - r * kSolveBlock;
    u_lds[idx] = c < count ? sp.U[(size_t)(sp.i1 + r) * K + sp.i1 + c] : 0.f;
  }
  __syncthreads();
  const int row = blockIdx.x * kSolveWaves + wave;
  if (row >= sp.rows) return;
  float* wrow = sp.W + (size_t)row * K;
  const int c0 = lane, c1 = lane + 64;
  float w0 = c0 < count ? wrow[sp.i1 + c0] : 0.f;
  float w1 = c1 < count ? wrow[sp.i1 + c1] : 0.f;
  // the range of a group is taken from the values the block started with (the reference reads
  // them from the matrix that only receives the updates of finished blocks)
  const float w0s = w0, w1s = w1;
  float q0 = 0.f, q1 = 0.f, e0 = 0.f, e1 = 0.f, loss = 0.f;
  float scale = 1.f, zero = 0.f;
  const int gs = sp.groupsize;
  if (gs <= 0) {
    scale = sp.scale[row];
    zero = sp.zero[row];
  } else if (sp.i1 % gs != 0) {
    // the block starts inside a group (groups longer than a block): its parameters were
    // found when the group started
    const int g = sp.i1 / gs;
    scale = sp.scale[(size_t)row * sp.G + g];
    zero = sp.zero[(size_t)row * sp.G + g];
  }
  for (int i = 0; i < count; ++i) {
    const int col = sp.i1 + i;
    if (gs > 0 && col % gs == 0 && sp.given) {
      scale = sp.scale[(size_t)row * sp.G + col / gs];
      zero = sp.zero[(size_t)row * sp.G + col / gs];
    } else if (gs > 0 && col % gs == 0) {
      // range of the group's values: the block's part as it was at block entry, the rest from W
      const int end = min(col + gs, K);       // one past the group's last column
      const int in_block = min(end - sp.i1, count);
      float lo = 0.f, hi = 0.f;              // the reference's range always contains 0
      if (c0 >= i && c0 < in_block) { lo = fminf(lo, w0s); hi = fmaxf(hi, w0s); }
      if (c1 >= i && c1 < in_block) { lo = fminf(lo, w1s); hi = fmaxf(hi, w1s); }
      for (int c = sp.i1 + count + lane; c < end; c += 64) {
        const float v = wrow[c];
        lo = fminf(lo, v);
        hi = fmaxf(hi, v);
      }
      lo = wave_min(lo);
      hi = wave_max(hi);
      if (sp.sym) {
        hi = fmaxf(fabsf(lo), hi);
        if (lo < 0.f) lo = -hi;
      }
      if (lo == 0.f && hi == 0.f) { lo = -1.f; hi = 1.f; }
      scale = __fdiv_rn(__fsub_rn(hi, lo), 15.f);
      zero = sp.sym ? 8.f : rintf(__fdiv_rn(-lo, scale));
      if (lane == 0) {
        sp.scale[(size_t)row * sp.G + col / gs] = scale;
        sp.zero[(size_t)row * sp.G + col / gs] = zero;
      }
    }
    const float wi = __shfl(i < 64 ? w0 : w1, i & 63, 64);
    const float d = u_lds[i * kSolveBlock + i];
    float q = rintf(__fdiv_rn(wi, scale)) + zero;
    q = fminf(fmaxf(q, 0.f), 15.f);
    const float qf = __fmul_rn(scale, __fsub_rn(q, zero));
    const float diff = __fsub_rn(wi, qf);
    const float err = __fdiv_rn(diff, d);
    loss += __fdiv_rn(__fmul_rn(diff, diff), __fmul_rn(d, d));
    if (i < 64) {
      if (lane == i) { q0 = qf; e0 = err; }
      if (c0 > i) w0 = __fsub_rn(w0, __fmul_rn(err, u_lds[i * kSolveBlock + c0]));
    } else if (lane == i - 64) {
      q1 = qf; e1 = err;
    }
    if (c1 > i) w1 = __fsub_rn(w1, __fmul_rn(err, u_lds[i * kSolveBlock + c1]));
  }
  float* qrow = sp.Q + (size_t)row * K + sp.i1;
  float* erow = sp.Err + (size_t)row * kSolveBlock;
  if (c0 < count) { qrow[c0] = q0; erow[c0] = e0; } else erow[c0] = 0.f;
  if (c1 < count) { qrow[c1] = q1; erow[c1] = e1; } else erow[c1] = 0.f;
  if (lane == 0) sp.loss[row] += 0.5f * loss;
}

}  // namespace q4

namespace q4host {

int launch_gptq_solve_block(float* W, const float* U, float* Q, float* Err, float* loss, float* scale, float* zero,
                            int rows, int K, int i1, int count, int groupsize, int G, int sym, hipStream_t stream) {
  q4::SolveParams sp{W, U, Q, Err, loss, scale, zero, rows, K, i1, count, groupsize, G, sym & 1, (sym >> 1) & 1};
  const size_t smem = (size_t)count * q4::kSolveBlock * sizeof(float);
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)q4::gptq_solve_block_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                              (int)smem);
  hipLaunchKernelGGL(q4::gptq_solve_block_kernel, dim3((unsigned)((rows + q4::kSolveWaves - 1) / q4::kSolveWaves)),
                     dim3(64 * q4::kSolveWaves), smem, stream, sp);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_gptq_solve_block: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
