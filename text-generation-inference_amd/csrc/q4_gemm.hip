// Prefill path, host side: tile and split-K plan, launch of the GPTQ MFMA kernel and of the
// split-K reduction.  The device code is in q4_gemm_kernels.cuh.
#include "q4_gemm_kernels.cuh"
#include "q4_gemm_wide.cuh"

namespace q4host {

using q4::GemmParams;
using q4::Problem;

bool gemm_supported(const q4_weight* w, int M, int dtype) {
  (void)dtype;
  if (w->layout != Q4_LAYOUT_GPTQ || w->g_idx != nullptr) return false;
  if (M < 1) return false;
  if (w->K % q4::kBK != 0 || w->N % 128 != 0) return false;
  const int gs = w->groupsize;
  if (!(gs == 32 || (gs >= 64 && gs % 64 == 0))) return false;
  if ((long)w->num_groups * gs < w->K) return false;
  // the kernel addresses weights, scales and activations through 32-bit byte offsets (launch_gemm
  // feeds longer activation matrices in row blocks)
  if ((long)w->K * w->N >= (1L << 33) || (long)w->num_groups * w->N >= (1L << 31) || w->K > (1 << 22)) return false;
  return true;
}

// rows of x a single launch may address: M * K * 2 bytes below 4 GB
static int gemm_max_rows(int K) {
  const long rows = ((1L << 31) - 1) / (K > 0 ? K : 1);
  return (int)(rows > (1L << 30) ? (1L << 30) : rows);
}

// two K groups per workgroup (eight waves)
template <int DTYPE, int BM>
static void launch_tile_kg2(const GemmParams& gp, int gs, dim3 grid, size_t smem, hipStream_t stream) {
  auto k = gs == 32 ? q4::gemm_gptq_kernel<DTYPE, BM, 2, 2, false, 2> : q4::gemm_gptq_kernel<DTYPE, BM, 1, 2, false, 2>;
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, dim3(512), smem, stream, gp);
}

template <int DTYPE, int BM, int NW>
static void launch_tile(const GemmParams& gp, int gs, dim3 grid, size_t smem, hipStream_t stream) {
  using namespace q4;
  if (gs == 32) {
    auto k = gemm_gptq_kernel<DTYPE, BM, 2, NW>;
    if (smem > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(256), smem, stream, gp);
  } else {
    auto k = gemm_gptq_kernel<DTYPE, BM, 1, NW>;
    if (smem > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(256), smem, stream, gp);
  }
}

// gated-MLP epilogue: 128 gate + 128 up columns per workgroup, groups of at least 64 rows
template <int DTYPE, int BM>
static void launch_tile_fused(const GemmParams& gp, dim3 grid, size_t smem, hipStream_t stream) {
  auto k = q4::gemm_gptq_kernel<DTYPE, BM, 1, 2, false, 1, true>;
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, dim3(256), smem, stream, gp);
}

// Tile shape and split factor for a problem; shared by the launcher and the workspace sizing.
struct GemmPlan {
  int bm, nw, splits;
  int kg = 1;  // K groups per workgroup (2: eight waves, see gemm_gptq_kernel)
  long tiles;
};

static GemmPlan gemm_plan(int M, int K, int N) {
  // Tile choice (all with 4 waves side by side along N):
  //   128 x 256  the default; two workgroups per CU once there are more than 256 of them (a
  //              256 x 256 tile with one wave per SIMD measured 0..12 % slower on every Llama-3-8B
  //              projection at M = 512 .. 4096: 4096 x 28672 at M = 2048 501 against 446 us);
  //    64 x 256  up to 64 rows: half the accumulators, three workgroups per CU keep more weight
  //              loads in flight (4096 x 28672 at M = 32: 30.6 against 40.7 us; 8192 x 8192:
  //              23.4 against 28.5 us); a cost model of its own for the split factor measured
  //              no better than the 128-row one;
  //   128 x 128  only when N is not a multiple of 256 (measured slower than 128 x 256
  //              everywhere else: twice the activation-fragment reads per MFMA).
  GemmPlan g;
  const bool n256 = N % 256 == 0;
  g.bm = 128;
  g.nw = n256 ? 2 : 1;
  if (M <= 64 && n256) g.bm = 64;
  const int bn = 128 * g.nw;
  g.tiles = (long)((M + g.bm - 1) / g.bm) * (N / bn);
  // Split-K when the tiles alone leave CUs idle (one workgroup runs the whole K loop at
  // ~0.9 us per 64-row K tile whatever M is: 14336 x 4096 took 200 us for every M up to
  // 1024).  Aim at two workgroups per CU, keep at least 8 K tiles per workgroup.
  // The split factor minimises a cost model fitted to measurements on MI355X: a workgroup
  // takes ~0.9 us per K tile alone on its CU and ~1.3 us when two share one; the partial
  // tiles cost a second launch (~5 us) plus S * M * N * 8 bytes of traffic at ~5 TB/s.
  // (4096 x 6144 at M = 1024: 70 us unsplit, 86 us with three splits; 14336 x 4096 at
  // M = 512: 200 us unsplit, 78 us with eight.)
  g.splits = 1;
  if (g.bm <= 128 && g.tiles < 256) g.splits = gemm_pick_splits(g.tiles, K / q4::kBK, M, N, 0.9, 1.3);
  // One workgroup per CU (the tiles, times the split factor, do not exceed the CU count): eight
  // waves in two K groups put two waves on every SIMD.  Measured at M = 2048 on MI355X:
  // 4096 x 4096 77.8 -> 70.2 us, 14336 x 4096 296 -> 246 us; with more workgroups than CUs the
  // four-wave kernel, two to a CU, is the faster one (4096 x 6144: 115 against 127 us).
  if (g.bm == 128 && g.nw == 2 && g.tiles * g.splits <= 256 && (K / q4::kBK) % (2 * g.splits) == 0) g.kg = 2;
  return g;
}

// The 128 x 384 tile (gemm_gptq_wide_kernel, one workgroup of eight waves per CU) against the
// 128 x 256 tile (two workgroups of four waves per CU): taken when the narrower tile runs unsplit
// in a single, partly filled round of its 512 workgroup slots and the wide one fills its round of
// 256 clearly better.  4096 x 6144: M = 2048, 384 tiles of 128 x 256 (half of the CUs with a
// single workgroup) against 256 of 128 x 384, 110.4 -> 106.4 us; M = 1536, 288 against 192 tiles,
// 96.3 -> 84.1 us.
static bool gemm_wide_plan(const q4_weight* w, int M, const GemmPlan& g) {
  if (w->N % q4::kWideBN != 0 || w->groupsize < 64 || w->groupsize % 64 != 0) return false;
  if (g.bm != 128 || g.nw != 2 || g.splits != 1 || g.kg != 1) return false;
  if ((long)(w->K >> 3) * w->N * 4 >= (1L << 32)) return false;
  const long wide = (long)((M + 127) / 128) * (w->N / q4::kWideBN);
  if (g.tiles <= 256 || g.tiles >= 512 || wide > 256) return false;  // one round of either (two: 191 against 182 us at M = 4096)
  return (double)wide / 256.0 >= (double)g.tiles / 512.0 + 0.15;
}

template <int DTYPE>
static void launch_wide(const GemmParams& gp, dim3 grid, hipStream_t stream) {
  hipLaunchKernelGGL(q4::gemm_gptq_wide_kernel<DTYPE>, grid, dim3(512), 2 * q4::kWideBM * q4::kDirectRowBytes, stream, gp);
}

// per_cu: workgroups of this kernel that fit on a CU together (1 or 2)
int gemm_pick_splits(long tiles, int KT, int M, int N, double us_alone, double us_shared, int per_cu) {
  static const int kCandidates[] = {1, 2, 3, 4, 6, 8, 12, 16};
  double best = -1.0;
  int splits = 1;
  for (int sp : kCandidates) {
    if (sp > 1 && KT / sp < 8) break;  // at least 8 K tiles (512 rows) per workgroup
    const long wgs = tiles * sp;
    const long slots = 256L * per_cu;
    const long rounds = (wgs + slots - 1) / slots;
    const double per_tile = (per_cu == 1 || wgs <= 256) ? us_alone : us_shared;
    double t = (double)rounds * ((KT + sp - 1) / sp) * per_tile;
    if (sp > 1) t += 5.0 + (double)sp * M * N * 8.0 / 5.0e6;
    if (best < 0.0 || t < best) {
      best = t;
      splits = sp;
    }
  }
  return splits;
}

void launch_gemm_reduce(const float* partials, const void* bias, void* y, int M, int N, int splits, int dtype,
                        hipStream_t stream) {
  const long quads = (long)M * (N / 4);
  long blocks = (quads + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (dtype == Q4_DTYPE_F16)
    hipLaunchKernelGGL(q4::gemm_reduce_kernel<Q4_DTYPE_F16>, dim3((unsigned)blocks), dim3(256), 0, stream, partials,
                       bias, (uint16_t*)y, M, N, splits);
  else
    hipLaunchKernelGGL(q4::gemm_reduce_kernel<Q4_DTYPE_BF16>, dim3((unsigned)blocks), dim3(256), 0, stream, partials,
                       bias, (uint16_t*)y, M, N, splits);
}

// fp32 partial tiles of the split-K variants: splits x M x N floats (upper bound over the
// GPTQ kernel and the AWQ / act-order kernel, whose tiles differ).
size_t gemm_workspace_bytes(int M, int K, int N) {
  if (K % q4::kBK != 0 || N % 128 != 0) return 0;
  // the GPTQ kernel runs from 17 rows on; the AWQ / act-order kernel may be forced at any M and
  // is dispatched from 9 rows on for small AWQ layers
  int splits = M > 16 ? gemm_plan(M, K, N).splits : 1;
  for (const bool one_per_cu : {false, true}) {
    const int other = gemm_awq_splits(M, K, N, one_per_cu);
    if (other > splits) splits = other;
  }
  {
    const int other = gemm_awq_splits(M, K, N, true, true);  // act-order, 256-row tiles
    if (other > splits) splits = other;
  }
  const size_t bytes = splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
  const size_t direct = gemm_awq_direct_workspace_bytes(M, K, N);
  return direct > bytes ? direct : bytes;
}

// The prefill kernel with the gated-MLP epilogue: one launch where the plain kernel would run
// unsplit (the fused tile cannot leave partial sums), groups of at least 64 rows.
bool gemm_gate_up_supported(const q4_weight* w, int M, int dtype) {
  if (!gemm_supported(w, M, dtype) || w->N % 512 != 0 || w->groupsize < 64 || M > gemm_max_rows(w->K)) return false;
  const GemmPlan g = gemm_plan(M, w->K, w->N);
  return g.splits == 1 && g.nw == 2 && g.bm <= 128;
}

int launch_gemm_gate_up(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype, int act,
                        hipStream_t stream) {
  using namespace q4;
  if (!gemm_gate_up_supported(w, M, dtype)) {
    set_error("q4_linear_gate_up(gemm): no fused prefill kernel for this problem (M=%d K=%d N=%d groupsize=%d)", M, w->K,
              w->N, w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  GemmParams gp;
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, nullptr, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  gp.p.gate_up_act = act + 1;
  gp.moe = q4::MoeView{};
  gp.partial_rows = M;
  gp.splits = 1;
  gp.partials = nullptr;
  const GemmPlan g = gemm_plan(M, w->K, w->N);
  size_t smem = 2 * (size_t)g.bm * kAUnitsPerRow * 16;
  const size_t exchange = (size_t)4 * (g.bm / 32) * 16 * 64 * 4;  // every wave's rounded tile
  if (exchange > smem) smem = exchange;
  dim3 grid((unsigned)g.tiles);
  if (dtype == Q4_DTYPE_F16) {
    if (g.bm == 64) launch_tile_fused<Q4_DTYPE_F16, 64>(gp, grid, smem, stream);
    else launch_tile_fused<Q4_DTYPE_F16, 128>(gp, grid, smem, stream);
  } else {
    if (g.bm == 64) launch_tile_fused<Q4_DTYPE_BF16, 64>(gp, grid, smem, stream);
    else launch_tile_fused<Q4_DTYPE_BF16, 128>(gp, grid, smem, stream);
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear_gate_up(gemm): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

int launch_gemm(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                void* workspace, size_t workspace_bytes, hipStream_t stream) {
  using namespace q4;
  if (!gemm_supported(w, M, dtype)) {
    set_error("q4_linear(gemm): unsupported problem (layout=%d g_idx=%p M=%d K=%d N=%d groupsize=%d)",
              w->layout, (const void*)w->g_idx, M, w->K, w->N, w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  if (M > gemm_max_rows(w->K)) {
    // beyond the 32-bit activation offsets of one launch: row blocks (a multiple of the tile height)
    const int block = gemm_max_rows(w->K) / 256 * 256;
    for (int m0 = 0; m0 < M; m0 += block) {
      const int rows = M - m0 < block ? M - m0 : block;
      const int rc = launch_gemm(w, (const uint16_t*)x + (size_t)m0 * w->K, bias, (uint16_t*)y + (size_t)m0 * w->N, rows, dtype,
                                 workspace, workspace_bytes, stream);
      if (rc != Q4_OK) return rc;
    }
    return Q4_OK;
  }
  GemmParams gp;
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, nullptr, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  gp.moe = q4::MoeView{};
  gp.partial_rows = M;
  GemmPlan g = gemm_plan(M, w->K, w->N);
  // without room for the partial tiles every workgroup owns a whole tile (slower, same result
  // up to fp32 summation order)
  const size_t partial_bytes = (size_t)g.splits * M * w->N * sizeof(float);
  if (g.splits > 1 && (workspace == nullptr || workspace_bytes < Q4_WORKSPACE_COUNTER_BYTES + partial_bytes))
    g.splits = 1;
  gp.splits = g.splits;
  gp.partials = g.splits > 1 ? (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES) : nullptr;
  if (gemm_wide_plan(w, M, g)) {
    const long wide = (long)((M + 127) / 128) * (w->N / kWideBN);
    if (dtype == Q4_DTYPE_F16) launch_wide<Q4_DTYPE_F16>(gp, dim3((unsigned)wide), stream);
    else launch_wide<Q4_DTYPE_BF16>(gp, dim3((unsigned)wide), stream);
    const hipError_t werr = hipGetLastError();
    if (werr != hipSuccess) {
      set_error("q4_linear(gemm): launch failed: %s", hipGetErrorString(werr));
      return Q4_ERR_LAUNCH;
    }
    return Q4_OK;
  }
  const int bm = g.bm, nw = g.nw;
  const long total = g.tiles * g.splits;
  if (total > 0x7fffffffL) {
    set_error("q4_linear(gemm): grid too large");
    return Q4_ERR_UNSUPPORTED;
  }
  size_t smem = 2 * (size_t)bm * kAUnitsPerRow * 16;
  dim3 grid((unsigned)total);
  const int gs = w->groupsize;
  const bool kg2 = g.kg == 2 && nw == 2 && bm <= 128 && (w->K / kBK) % (2 * g.splits) == 0;
  if (kg2) {
    smem *= 2;
    const size_t xch = (size_t)(bm / 32) * 2 * 16 * 256 * sizeof(float);
    if (xch > smem) smem = xch;
    if (dtype == Q4_DTYPE_F16) {
      if (bm == 64) launch_tile_kg2<Q4_DTYPE_F16, 64>(gp, gs, grid, smem, stream);
      else launch_tile_kg2<Q4_DTYPE_F16, 128>(gp, gs, grid, smem, stream);
    } else {
      if (bm == 64) launch_tile_kg2<Q4_DTYPE_BF16, 64>(gp, gs, grid, smem, stream);
      else launch_tile_kg2<Q4_DTYPE_BF16, 128>(gp, gs, grid, smem, stream);
    }
  } else if (dtype == Q4_DTYPE_F16) {
    if (bm == 64) launch_tile<Q4_DTYPE_F16, 64, 2>(gp, gs, grid, smem, stream);
    else if (nw == 2) launch_tile<Q4_DTYPE_F16, 128, 2>(gp, gs, grid, smem, stream);
    else launch_tile<Q4_DTYPE_F16, 128, 1>(gp, gs, grid, smem, stream);
  } else {
    if (bm == 64) launch_tile<Q4_DTYPE_BF16, 64, 2>(gp, gs, grid, smem, stream);
    else if (nw == 2) launch_tile<Q4_DTYPE_BF16, 128, 2>(gp, gs, grid, smem, stream);
    else launch_tile<Q4_DTYPE_BF16, 128, 1>(gp, gs, grid, smem, stream);
  }
  if (g.splits > 1) launch_gemm_reduce(gp.partials, bias, y, M, w->N, g.splits, dtype, stream);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemm): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
