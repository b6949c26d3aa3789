// Prefill path for the AWQ layout, host side: tile / split-K plan and launch of the kernel that
// unpacks the checkpoint words in registers (q4_gemm_awq_direct.cuh).
#include "q4_gemm_awq_direct.cuh"

namespace q4host {

using q4::GemmParams;
using q4::Problem;

bool gemm_awq_direct_supported(const q4_weight* w, int M, int dtype) {
  (void)dtype;
  if (w->layout != Q4_LAYOUT_AWQ || w->g_idx != nullptr) return false;
  if (M < 1) return false;
  if (w->K % q4::kBK != 0 || w->N % 256 != 0) return false;
  // buffer descriptors with 32-bit byte counts
  if ((long)M * w->K >= (1L << 30) || (long)w->K * w->N >= (1L << 32)) return false;
  if (w->groupsize < 64 || w->groupsize % 64 != 0) return false;  // one group per 64-row K tile
  return (long)w->num_groups * w->groupsize >= w->K;
}

struct DirectPlan {
  int bm, splits, kg;
  long tiles;
};

static DirectPlan direct_plan(int M, int K, int N) {
  DirectPlan g;
  // Row tile: 96 rows (the largest whose accumulators leave the unpacking free of register
  // spills) unless 64-row tiles cover M with much less padding (M = 128: 34.8 against 38.5 us
  // on 4096 x 14336; from M = 256 on the larger tile wins or ties); 64 and 32 rows below that.
  g.bm = M <= 32 ? 32 : (M <= 64 ? 64 : 96);
  if (g.bm == 96 && (long)((M + 95) / 96) * 96 * 5 > (long)((M + 63) / 64) * 64 * 6) g.bm = 64;
  // Several rounds of the chip: a CU works through ceil(tiles / 256) tiles whatever their height
  // (two 96-row or three 64-row workgroups per CU take the same time per row), so the smaller
  // tile wins where it leaves clearly fewer rows to the busiest CU (14336 x 4096 or 4096 x 4096
  // at M = 2048: 352 tiles of 96 rows against 512 of 64; 310 -> 274 us and 89 -> 83 us).
  if (g.bm == 96) {
    const long cols = N / 256;
    const long t96 = (long)((M + 95) / 96) * cols, t64 = (long)((M + 63) / 64) * cols;
    if (t96 > 256 && ((t64 + 255) / 256) * 64 * 4 <= ((t96 + 255) / 256) * 96 * 3) g.bm = 64;
  }
  g.tiles = (long)((M + g.bm - 1) / g.bm) * (N / 256);
  g.splits = 1;
  g.kg = 1;
  const int KT = K / q4::kBK;
  // under-filled grids: same cost model as the GPTQ kernel (a workgroup walks its K tiles at a
  // rate that hardly depends on M; partial tiles cost a second launch and their traffic)
  if (g.tiles < 256) g.splits = gemm_pick_splits(g.tiles, KT, M, N, 0.9, 1.3);
  // one workgroup per CU: eight waves in two K groups put two waves on every SIMD
  if (g.bm == 96 && g.tiles * g.splits <= 256 && KT % (2 * g.splits) == 0) g.kg = 2;
  return g;
}

size_t gemm_awq_direct_workspace_bytes(int M, int K, int N) {
  if (K % q4::kBK != 0 || N % 256 != 0) return 0;
  const int splits = direct_plan(M, K, N).splits;
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

template <int DTYPE, int BM, int KG>
static void launch_direct(const GemmParams& gp, dim3 grid, size_t smem, hipStream_t stream) {
  auto k = q4::gemm_awq_direct_kernel<DTYPE, BM, KG>;
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, dim3(256 * KG), smem, stream, gp);
}

int launch_gemm_awq_direct(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                           void* workspace, size_t workspace_bytes, hipStream_t stream) {
  using namespace q4;
  if (!gemm_awq_direct_supported(w, M, dtype)) {
    set_error("q4_linear(gemm/awq): unsupported problem for the register-unpack kernel (M=%d K=%d N=%d groupsize=%d)",
              M, w->K, w->N, w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  GemmParams gp;
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, nullptr, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  gp.moe = q4::MoeView{};
  gp.partial_rows = M;
  DirectPlan g = direct_plan(M, w->K, w->N);
  const size_t partial_bytes = (size_t)g.splits * M * w->N * sizeof(float);
  if (g.splits > 1 && (workspace == nullptr || workspace_bytes < Q4_WORKSPACE_COUNTER_BYTES + partial_bytes)) {
    g.splits = 1;  // no room for partial tiles: every workgroup owns a whole tile
    g.kg = (g.bm == 96 && g.tiles <= 256 && (w->K / kBK) % 2 == 0) ? 2 : 1;
  }
  gp.splits = g.splits;
  gp.partials = g.splits > 1 ? (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES) : nullptr;
  const long total = g.tiles * g.splits;
  if (total > 0x7fffffffL) {
    set_error("q4_linear(gemm/awq): grid too large");
    return Q4_ERR_UNSUPPORTED;
  }
  size_t smem = 2 * (size_t)g.bm * kDirectRowBytes;
  const dim3 grid((unsigned)total);
  auto launch_dt = [&](auto dt) {
    constexpr int DT = decltype(dt)::value;
    if (g.kg == 2) {
      smem *= 2;
      const size_t xch = (size_t)(g.bm / 16) * 4 * 4 * 256 * sizeof(float);  // one accumulator set
      if (xch > smem) smem = xch;
      launch_direct<DT, 96, 2>(gp, grid, smem, stream);
    } else if (g.bm == 32) {
      launch_direct<DT, 32, 1>(gp, grid, smem, stream);
    } else if (g.bm == 64) {
      launch_direct<DT, 64, 1>(gp, grid, smem, stream);
    } else {
      launch_direct<DT, 96, 1>(gp, grid, smem, stream);
    }
  };
  if (dtype == Q4_DTYPE_F16) launch_dt(std::integral_constant<int, Q4_DTYPE_F16>{});
  else launch_dt(std::integral_constant<int, Q4_DTYPE_BF16>{});
  if (g.splits > 1) launch_gemm_reduce(gp.partials, bias, y, M, w->N, g.splits, dtype, stream);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemm/awq): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
