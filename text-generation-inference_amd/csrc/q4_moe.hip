// Mixture of experts: routing, the grouped (per-expert) linear layer and the weighted sum.
//
// The rows of the grouped problem are the (token, expert) pairs sorted by expert.  Nothing
// on this path needs the host to know how many rows an expert received:
//   * moe_route_kernel (one workgroup) computes softmax -> top-k -> renormalisation per token
//     and counting-sorts the pairs by expert with LDS atomics;
//   * the grouped linear layer launches the ordinary decode or prefill kernel once more per
//     expert (a grid dimension); every workgroup reads its expert's row range from device
//     memory, narrows the problem to it and leaves at once when the range is empty or ends
//     before its tile.  The decode kernel therefore streams the packed weights of exactly
//     the experts that were chosen, once per 16 rows they received;
//   * moe_combine_kernel adds the topk rows of every token, weighted, in fp32.
#include "q4_gemm_kernels.cuh"
#include "q4_gemv_kernels.cuh"

namespace q4 {

constexpr int kMoeMaxExperts = 256;
constexpr int kMoeMaxTopk = 8;

template <int GDT>
__device__ __forceinline__ float load_logit(const void* g, size_t i) {
  if constexpr (GDT == Q4_DTYPE_F16) return (float)((const half_t*)g)[i];
  else if constexpr (GDT == Q4_DTYPE_BF16) return bf16_bits_to_f32(((const uint16_t*)g)[i]);
  else return ((const float*)g)[i];
}

// groups > 0: grouped top-k -- the experts form `groups` equal groups, a token keeps the
// `topk_group` groups with the largest member and chooses its experts among those only.
template <int GDT>
__global__ __launch_bounds__(1024) void moe_route_kernel(const void* __restrict__ gating, int T, int E, int topk,
                                                         int renormalize, int groups, int topk_group,
                                                         float* __restrict__ topk_weights,
                                                         int32_t* __restrict__ topk_ids,
                                                         int32_t* __restrict__ sorted_tokens,
                                                         int32_t* __restrict__ pair_slot,
                                                         int32_t* __restrict__ expert_offsets) {
  __shared__ int count[kMoeMaxExperts];
  __shared__ int cursor[kMoeMaxExperts];
  // logits of a batch of tokens, staged with coalesced loads: a thread that walks its token's
  // row in global memory pays a memory round trip per expert
  constexpr int kStage = 8192;
  __shared__ float logits[kStage];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += blockDim.x) count[e] = 0;
  __syncthreads();

  const int batch = kStage / E;  // tokens per staged batch (E <= 256)
  for (int t0 = 0; t0 < T; t0 += batch) {
    const int nt = min(batch, T - t0);
    for (int i = tid; i < nt * E; i += blockDim.x) logits[i] = load_logit<GDT>(gating, (size_t)t0 * E + i);
    __syncthreads();
    // ---- per token: softmax over the experts in fp32, the topk largest (ties: lowest index)
    for (int tl = tid; tl < nt; tl += blockDim.x) {
      const int t = t0 + tl;
      const float* lg = logits + tl * E;
      float mx = lg[0];
      for (int e = 1; e < E; ++e) mx = fmaxf(mx, lg[e]);
      float sum = 0.f;
      for (int e = 0; e < E; ++e) sum += expf(lg[e] - mx);
      // groups a token may choose from, as a bit mask (softmax is monotonic: logits decide)
      uint32_t allowed = 0xFFFFFFFFu;
      const int per_group = groups > 0 ? E / groups : E;
      if (groups > 0) {
        allowed = 0u;
        for (int j = 0; j < topk_group; ++j) {
          int best = -1;
          float bv = 0.f;
          for (int g = 0; g < groups; ++g) {
            if ((allowed >> g) & 1u) continue;
            float gm = lg[g * per_group];
            for (int e = 1; e < per_group; ++e) gm = fmaxf(gm, lg[g * per_group + e]);
            if (best < 0 || gm > bv) {
              best = g;
              bv = gm;
            }
          }
          allowed |= 1u << best;
        }
      }
      // no per-thread arrays (they would live in scratch memory): a chosen expert is struck
      // from the staged row, ids and weights go straight to their output
      float* row_lg = logits + tl * E;
      float wsum = 0.f;
      for (int j = 0; j < topk; ++j) {
        int best = -1;
        float bv = 0.f;
        for (int e = 0; e < E; ++e) {
          if (groups > 0 && !((allowed >> (e / per_group)) & 1u)) continue;
          const float v = row_lg[e];
          if (v == -INFINITY) continue;  // taken (or never eligible)
          if (best < 0 || v > bv) {
            best = e;
            bv = v;
          }
        }
        if (best < 0) best = 0;  // every logit -inf: keep the indices in range
        const float pw = expf(bv - mx) / sum;
        wsum += pw;
        topk_ids[(size_t)t * topk + j] = best;
        topk_weights[(size_t)t * topk + j] = pw;
        row_lg[best] = -INFINITY;
        atomicAdd(&count[best], 1);
      }
      if (renormalize) {
        for (int j = 0; j < topk; ++j) topk_weights[(size_t)t * topk + j] /= wsum;
      }
    }
    __syncthreads();  // the batch is consumed before the next one overwrites it
  }
  __syncthreads();
  if (tid == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      expert_offsets[e] = run;
      cursor[e] = run;
      run += count[e];
    }
    expert_offsets[E] = run;
  }
  __syncthreads();
  // ---- scatter: every pair takes the next free row of its expert
  for (int t = tid; t < T; t += blockDim.x) {
    for (int j = 0; j < topk; ++j) {
      const int e = topk_ids[(size_t)t * topk + j];  // written above by this same thread
      const int slot = atomicAdd(&cursor[e], 1);
      sorted_tokens[slot] = t;
      pair_slot[(size_t)t * topk + j] = slot;
    }
  }
}

// out[t, n..n+7] = sum_j w[t, j] * y[slot(t, j), n..n+7]
template <int DTYPE>
__global__ __launch_bounds__(256) void moe_combine_kernel(const uint16_t* __restrict__ y,
                                                          const float* __restrict__ topk_weights,
                                                          const int32_t* __restrict__ pair_slot,
                                                          uint16_t* __restrict__ out, int topk, int N) {
  const int t = blockIdx.y;
  const int n = (blockIdx.x * 256 + threadIdx.x) * 8;
  if (n >= N) return;
  float acc[8] = {};
  for (int j = 0; j < topk; ++j) {
    const float w = topk_weights[(size_t)t * topk + j];
    const int slot = pair_slot[(size_t)t * topk + j];
    const uint4_t v = *(const uint4_t*)(y + (size_t)slot * N + n);
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float lo, hi;
      if constexpr (DTYPE == Q4_DTYPE_F16) {
        const half2_t h = as_half2(u[i]);
        lo = (float)h.x;
        hi = (float)h.y;
      } else {
        lo = bf16_bits_to_f32((uint16_t)(u[i] & 0xFFFFu));
        hi = bf16_bits_to_f32((uint16_t)(u[i] >> 16));
      }
      acc[2 * i] = fmaf(w, lo, acc[2 * i]);
      acc[2 * i + 1] = fmaf(w, hi, acc[2 * i + 1]);
    }
  }
  uint4_t o;
  o.x = (uint32_t)store_act<DTYPE>(acc[0]) | ((uint32_t)store_act<DTYPE>(acc[1]) << 16);
  o.y = (uint32_t)store_act<DTYPE>(acc[2]) | ((uint32_t)store_act<DTYPE>(acc[3]) << 16);
  o.z = (uint32_t)store_act<DTYPE>(acc[4]) | ((uint32_t)store_act<DTYPE>(acc[5]) << 16);
  o.w = (uint32_t)store_act<DTYPE>(acc[6]) | ((uint32_t)store_act<DTYPE>(acc[7]) << 16);
  *(uint4_t*)(out + (size_t)t * N + n) = o;
}

}  // namespace q4

namespace q4host {

// fused gated-MLP decode instantiations (q4_gemv_gate_up.hip)
void launch_gemv_gate_up(const q4::GemvParams& gp, int dtype, int rmax, bool static128, dim3 grid, dim3 block,
                         size_t smem, hipStream_t stream, bool grouped);

using q4::GemmParams;
using q4::GemvParams;
using q4::MoeView;
using q4::Problem;

namespace {

int validate_moe_weight(const q4_moe_weight* w, const char* who) {
  if (w == nullptr) {
    set_error("%s: null q4_moe_weight", who);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  const q4_weight& e0 = w->expert0;
  if (w->num_experts < 1 || w->num_experts > q4::kMoeMaxExperts) {
    set_error("%s: num_experts=%d must be in 1..%d", who, w->num_experts, q4::kMoeMaxExperts);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (e0.qweight == nullptr || e0.qzeros == nullptr || e0.scales == nullptr) {
    set_error("%s: null qweight/qzeros/scales", who);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (e0.K < 8 || e0.N < 8 || e0.K % 8 != 0 || e0.N % 8 != 0 || e0.groupsize < 1 || e0.num_groups < 1) {
    set_error("%s: bad geometry K=%d N=%d groupsize=%d num_groups=%d", who, e0.K, e0.N, e0.groupsize,
              e0.num_groups);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (e0.layout != Q4_LAYOUT_GPTQ && e0.layout != Q4_LAYOUT_AWQ) {
    set_error("%s: unknown layout %d", who, e0.layout);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (e0.layout == Q4_LAYOUT_AWQ && e0.g_idx != nullptr) {
    set_error("%s: g_idx is not defined for the AWQ layout", who);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (e0.g_idx == nullptr && (long)e0.num_groups * e0.groupsize < e0.K) {
    set_error("%s: %d groups of %d rows do not cover K=%d", who, e0.num_groups, e0.groupsize, e0.K);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  const long qw = (long)(e0.K / 8) * e0.N, qz = (long)e0.num_groups * (e0.N / 8), sc = (long)e0.num_groups * e0.N;
  if (w->qweight_stride < qw || w->qzeros_stride < qz || w->scales_stride < sc ||
      (e0.g_idx != nullptr && w->g_idx_stride < e0.K)) {
    set_error("%s: expert strides (%lld, %lld, %lld) smaller than one expert (%ld, %ld, %ld)", who,
              (long long)w->qweight_stride, (long long)w->qzeros_stride, (long long)w->scales_stride, qw, qz, sc);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return Q4_OK;
}

// Decode plan of a grouped launch: the single-matrix configuration for the same row count,
// with the cross-workgroup K split divided by the number of experts expected to be active
// (their workgroups fill the chip together).
struct MoeGemvPlan {
  bool ok;
  GemvConfig cfg;
  int ntiles, mchunks, rows, kr_max;
  size_t slab_bytes, smem;
};

// The decode kernel takes 16 rows of an expert per workgroup; an expert can receive every
// token, so the grid has ceil(tokens / 16) row blocks per expert, of which those past the
// expert's count leave at once.  Each further block of an expert re-reads its weights (from
// L2 where it can).  Measured on Mixtral shapes (8 experts, top-2), decode against MFMA
// kernel: 4096 x 28672 113 / 268 us at 17 tokens, 163 / 240 us at 64; 14336 x 4096 (few
// column tiles, long K: the MFMA kernel splits K) 106 / 110 us at 17 tokens, 194 / 108 us
// at 64.  So the contiguous-group decode kernel is kept up to 64 tokens for K <= 8192 and up
// to 16 beyond; the act-order and AWQ decode kernels, whose cost per row is higher, up to 16.
constexpr int kMoeDecodeMaxTokens = 64;
constexpr int kMoeDecodeMaxTokensLongK = 16;

// gate_up: the kernel with the gated-MLP epilogue (one or two tokens, groups of whole chunks)
MoeGemvPlan moe_gemv_plan(const q4_moe_weight* w, int tokens, int topk, int dtype, bool gate_up = false) {
  using namespace q4;
  MoeGemvPlan pl{};
  const q4_weight* e0 = &w->expert0;
  const bool awq = e0->layout == Q4_LAYOUT_AWQ;
  const bool act = !awq && e0->g_idx != nullptr;
  const int rows = tokens < kRowsPerBlock ? tokens : kRowsPerBlock;
  const int max_tokens = (awq || act || e0->K > 8192) ? kMoeDecodeMaxTokensLongK : kMoeDecodeMaxTokens;
  if (tokens > max_tokens || !gemv_supported(e0, rows, dtype)) return pl;
  // fused epilogue: one token only (Mixtral gate_up, two experts: 33.5 us fused against 36.4 us with the
  // separate activation kernel; two tokens, four experts: 46.0 against 40.7 us)
  if (gate_up && (tokens > 1 || !gemv_gate_up_supported(e0, tokens, dtype))) return pl;
  const int mchunks = (tokens + kRowsPerBlock - 1) / kRowsPerBlock;
  GemvConfig cfg = gemv_pick_config(e0, rows, gate_up);
  cfg.words = gate_up ? 8 : 4;
  const int wave_cols = awq ? 256 : (gate_up ? 128 : 64);
  if (e0->N % (wave_cols * cfg.wcol) != 0) cfg.wcol = 1;
  const int kchunks = e0->K / 128;
  if (e0->N % wave_cols != 0 || cfg.wcol * cfg.wk > 8 || cfg.wk > kchunks) return pl;
  long active = (long)tokens * topk;
  if (active > w->num_experts) active = w->num_experts;
  const int max_splits = kchunks / cfg.wk;
  int splits = (int)(cfg.splits / active);
  if (splits < 1) splits = 1;
  // prefer a count that deals the 128-row chunks out evenly
  while (splits > 1 && kchunks % (splits * cfg.wk) != 0) --splits;
  const int ntiles = e0->N / (wave_cols * cfg.wcol);
  const bool tickets_fit = (long)ntiles * mchunks * w->num_experts <= Q4_WORKSPACE_TICKET_BYTES / 4;
  if (!tickets_fit) splits = 1;
  // LDS: the activation slab of `rows` x (largest K range of a workgroup), for act-order also
  // the g_idx slice and the parameter table; the wk waves' partial sums reuse it.  Split
  // further if it does not fit.
  const size_t smem_limit = 160 * 1024 - 1024;
  const int nt = awq ? 16 : (gate_up ? 8 : 4);
  auto kr_of = [&](int sp) {
    const long slots = (long)sp * cfg.wk;
    return (size_t)((kchunks * cfg.wk + slots - 1) / slots) * 128;  // upper bound of a workgroup's range
  };
  auto slab_of = [&](int sp) { return ((size_t)rows * (kr_of(sp) * 2 + 16) + 15) & ~(size_t)15; };
  auto smem_of = [&](int sp) {
    size_t bytes = slab_of(sp);
    if (act) bytes += ((kr_of(sp) * 2 + 15) & ~(size_t)15) + (size_t)e0->num_groups * 64 * cfg.wcol * 4;
    const size_t red = (size_t)(cfg.wk - 1) * cfg.wcol * nt * 4 * 64 * sizeof(float);
    return bytes > red ? bytes : red;
  };
  while (smem_of(splits) > smem_limit) {
    if (splits >= max_splits || !tickets_fit) return pl;
    ++splits;
  }
  pl.kr_max = (int)kr_of(splits);
  cfg.splits = splits;
  pl.ok = true;
  pl.cfg = cfg;
  pl.ntiles = ntiles;
  pl.mchunks = mchunks;
  pl.rows = rows;
  pl.slab_bytes = slab_of(splits);
  pl.smem = smem_of(splits);
  return pl;
}

template <typename Kernel>
void launch_with_smem(Kernel k, dim3 grid, dim3 block, size_t smem, hipStream_t stream, const GemvParams& gp) {
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, block, smem, stream, gp);
}

template <int DTYPE>
void launch_moe_gemv_dtype(const q4_weight* e0, dim3 grid, dim3 block, size_t smem, hipStream_t stream,
                           const GemvParams& gp) {
  using namespace q4;
  const int gs = e0->groupsize;
  if (e0->layout == Q4_LAYOUT_AWQ) {
    launch_with_smem(gemv_awq_kernel<DTYPE, 4, true>, grid, block, smem, stream, gp);
    return;
  }
  if (e0->g_idx != nullptr) {
    launch_with_smem(gemv_gptq_act_kernel<DTYPE, 4, true>, grid, block, smem, stream, gp);
    return;
  }
  if (gs == 128) launch_with_smem(gemv_gptq_kernel<DTYPE, 4, 4, true, 4, false, true>, grid, block, smem, stream, gp);
  else if (gs > 128) launch_with_smem(gemv_gptq_kernel<DTYPE, 4, 4, false, 4, false, true>, grid, block, smem, stream, gp);
  else if (gs == 64) launch_with_smem(gemv_gptq_kernel<DTYPE, 4, 2, false, 4, false, true>, grid, block, smem, stream, gp);
  else launch_with_smem(gemv_gptq_kernel<DTYPE, 4, 1, false, 4, false, true>, grid, block, smem, stream, gp);
}

template <int DTYPE, int BM, int NW>
void launch_moe_gemm_tile(int gs, dim3 grid, size_t smem, hipStream_t stream, const GemmParams& gp) {
  using namespace q4;
  if (gs == 32) hipLaunchKernelGGL((gemm_gptq_kernel<DTYPE, BM, 2, NW, true>), grid, dim3(256), smem, stream, gp);
  else hipLaunchKernelGGL((gemm_gptq_kernel<DTYPE, BM, 1, NW, true>), grid, dim3(256), smem, stream, gp);
}

// Row tile of the grouped MFMA launch: 64 rows while the experts receive at most 64 rows on
// average (three workgroups per CU keep more weight loads in flight), else 128.
int moe_gemm_bm(const q4_moe_weight* w, int tokens, int topk) {
  const long avg_rows = ((long)tokens * topk + w->num_experts - 1) / w->num_experts;
  return avg_rows <= 64 && w->expert0.N % 256 == 0 ? 64 : 128;
}

// Split-K factor of the grouped MFMA launch.  The host does not know the experts' row counts:
// it plans for an even spread (tokens * topk / experts rows each) and splits K when those
// tiles alone would leave CUs idle (Mixtral down projection at 64 tokens: 8 experts x 16
// column tiles, 224 K tiles each).
// the grouped GPTQ prefill kernel addresses the activation rows (tokens, or token-expert pairs)
// through 32-bit byte offsets
static bool moe_gemm_ok(const q4_weight* e0, int tokens, int topk, int dtype) {
  return gemm_supported(e0, tokens, dtype) && (long)tokens * topk * e0->K < (1L << 31);
}

int moe_gemm_splits(const q4_moe_weight* w, int tokens, int topk) {
  const q4_weight* e0 = &w->expert0;
  const long pairs = (long)tokens * topk;
  const long avg_rows = (pairs + w->num_experts - 1) / w->num_experts;
  const int nw = e0->N % 256 == 0 ? 2 : 1;
  const int bm = moe_gemm_bm(w, tokens, topk);
  const long tiles = (long)w->num_experts * ((avg_rows + bm - 1) / bm) * (e0->N / (128 * nw));
  if (tiles >= 256 || pairs > 0x7fffffffL) return 1;
  return gemm_pick_splits(tiles, e0->K / q4::kBK, (int)pairs, e0->N, 0.9, 1.3);
}

MoeView make_view(const q4_moe_weight* w, const int32_t* x_rows, const int32_t* offsets) {
  MoeView mv;
  mv.offsets = offsets;
  mv.x_rows = x_rows;
  mv.qweight_stride = (long)w->qweight_stride;
  mv.qzeros_stride = (long)w->qzeros_stride;
  mv.scales_stride = (long)w->scales_stride;
  mv.g_idx_stride = (long)w->g_idx_stride;
  return mv;
}

}  // namespace

// Upper bound over the kernels a grouped launch of this weight can take (for any dtype the
// plans are the same except that act-order bf16 has no decode kernel and goes to the MFMA one).
size_t moe_workspace_bytes(const q4_moe_weight* w, int tokens, int topk) {
  const q4_weight* e0 = &w->expert0;
  size_t partial_bytes = 0;
  auto take = [&](int splits) {
    const size_t b = splits > 1 ? (size_t)splits * tokens * topk * e0->N * sizeof(float) : 0;
    if (b > partial_bytes) partial_bytes = b;
  };
  for (const int dtype : {Q4_DTYPE_F16, Q4_DTYPE_BF16}) {
    const MoeGemvPlan plain = moe_gemv_plan(w, tokens, topk, dtype);
    const MoeGemvPlan fused = moe_gemv_plan(w, tokens, topk, dtype, true);
    if (plain.ok) take(plain.cfg.splits);
    if (fused.ok) take(fused.cfg.splits);
    if (!plain.ok) {
      if (moe_gemm_ok(e0, tokens, topk, dtype)) {
        take(moe_gemm_splits(w, tokens, topk));
      } else if (gemm_awq_supported(e0, tokens, dtype)) {
        const MoeLaunch ml{MoeView{}, w->num_experts, tokens, tokens * topk};
        const size_t b = gemm_awq_moe_workspace_bytes(e0, &ml);
        if (b > partial_bytes) partial_bytes = b;
      }
    }
  }
  return Q4_WORKSPACE_COUNTER_BYTES + partial_bytes;
}

// gate_up_act: 0 plain; Q4_ACT_* + 1: y[pairs, N / 2] = act(x @ gate) * (x @ up), decode kernel only
int launch_moe_linear(const q4_moe_weight* w, const void* x, const int32_t* x_rows, const int32_t* offsets, void* y,
                      int tokens, int topk, int dtype, void* workspace, size_t workspace_bytes, hipStream_t stream,
                      int gate_up_act = 0) {
  using namespace q4;
  const q4_weight* e0 = &w->expert0;
  const int pairs = tokens * topk;
  const MoeView mv = make_view(w, x_rows, offsets);
  const MoeGemvPlan pl = moe_gemv_plan(w, tokens, topk, dtype, gate_up_act != 0);
  if (gate_up_act != 0 && !pl.ok) {
    set_error("q4_moe_linear_gate_up: no fused kernel for tokens=%d K=%d N=%d groupsize=%d layout=%d", tokens, e0->K,
              e0->N, e0->groupsize, e0->layout);
    return Q4_ERR_UNSUPPORTED;
  }
  if (pl.ok) {
    const GemvConfig& cfg = pl.cfg;
    float* partials = nullptr;
    uint32_t* tickets = nullptr;
    if (cfg.splits > 1) {
      const size_t need = Q4_WORKSPACE_COUNTER_BYTES + (size_t)cfg.splits * pairs * e0->N * sizeof(float);
      if (workspace == nullptr || workspace_bytes < need) {
        set_error("q4_moe_linear: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
        return Q4_ERR_WORKSPACE;
      }
      tickets = (uint32_t*)workspace;
      partials = (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES);
    }
    GemvParams gp;
#ifdef Q4_PHASE_STAMPS
    gp.stamps = nullptr;  // (measurement builds stamp the dense launches only)
#endif
    gp.p = Problem{e0->qweight, e0->qzeros, (const half_t*)e0->scales, e0->g_idx, x, nullptr, y,
                   0,           e0->K,      e0->N,                     e0->groupsize, e0->num_groups};
    gp.p.gate_up_act = gate_up_act;
    gp.partials = partials;
    gp.tickets = tickets;
    gp.wcol = cfg.wcol;
    gp.wk = cfg.wk;
    gp.splits = cfg.splits;
    gp.cells = nullptr;
    gp.fixed_point_split = 0;
    gp.rows_per_block = kRowsPerBlock;
    gp.slab_stride = pl.kr_max * 2 + 16;
    gp.kr_max = pl.kr_max;
    gp.ntiles = pl.ntiles;
    (void)q4::set_k_deal(gp, e0->K / 128, cfg.splits, cfg.wk);
    gp.slab_bytes = (int)pl.slab_bytes;
    gp.partial_rows = pairs;
    gp.moe = mv;
    const dim3 grid((unsigned)(pl.ntiles * cfg.splits), (unsigned)pl.mchunks, (unsigned)w->num_experts);
    const dim3 block((unsigned)(64 * cfg.wcol * cfg.wk));
    if (gate_up_act != 0)
      launch_gemv_gate_up(gp, dtype, tokens <= 1 ? 1 : 2, e0->groupsize == 128, grid, block, pl.smem, stream, true);
    else if (dtype == Q4_DTYPE_F16) launch_moe_gemv_dtype<Q4_DTYPE_F16>(e0, grid, block, pl.smem, stream, gp);
    else launch_moe_gemv_dtype<Q4_DTYPE_BF16>(e0, grid, block, pl.smem, stream, gp);
  } else if (moe_gemm_ok(e0, tokens, topk, dtype)) {
    GemmParams gp;
    gp.p = Problem{e0->qweight, e0->qzeros, (const half_t*)e0->scales, nullptr, x, nullptr, y,
                   0,           e0->K,      e0->N,                     e0->groupsize, e0->num_groups};
    gp.p.gate_up_act = 0;
    int splits = moe_gemm_splits(w, tokens, topk);
    if (splits > 1 && (workspace == nullptr || workspace_bytes < Q4_WORKSPACE_COUNTER_BYTES +
                                                                     (size_t)splits * pairs * e0->N * sizeof(float)))
      splits = 1;  // no room for partial tiles
    gp.partials = splits > 1 ? (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES) : nullptr;
    gp.splits = splits;
    gp.partial_rows = pairs;
    gp.moe = mv;
    // an expert can receive every token: the grid covers `tokens` rows per expert
    const int nw = e0->N % 256 == 0 ? 2 : 1;
    const int bm = moe_gemm_bm(w, tokens, topk);
    const long tiles = (long)((tokens + bm - 1) / bm) * (e0->N / (128 * nw)) * splits;
    if (tiles > 0x7fffffffL || w->num_experts > 65535) {
      set_error("q4_moe_linear: grid too large");
      return Q4_ERR_UNSUPPORTED;
    }
    const dim3 grid((unsigned)tiles, (unsigned)w->num_experts);
    const size_t smem = 2 * (size_t)bm * kAUnitsPerRow * 16;
    if (dtype == Q4_DTYPE_F16) {
      if (bm == 64) launch_moe_gemm_tile<Q4_DTYPE_F16, 64, 2>(e0->groupsize, grid, smem, stream, gp);
      else if (nw == 2) launch_moe_gemm_tile<Q4_DTYPE_F16, 128, 2>(e0->groupsize, grid, smem, stream, gp);
      else launch_moe_gemm_tile<Q4_DTYPE_F16, 128, 1>(e0->groupsize, grid, smem, stream, gp);
    } else {
      if (bm == 64) launch_moe_gemm_tile<Q4_DTYPE_BF16, 64, 2>(e0->groupsize, grid, smem, stream, gp);
      else if (nw == 2) launch_moe_gemm_tile<Q4_DTYPE_BF16, 128, 2>(e0->groupsize, grid, smem, stream, gp);
      else launch_moe_gemm_tile<Q4_DTYPE_BF16, 128, 1>(e0->groupsize, grid, smem, stream, gp);
    }
    if (splits > 1) launch_gemm_reduce(gp.partials, nullptr, y, pairs, e0->N, splits, dtype, stream);
  } else if (gemm_awq_supported(e0, tokens, dtype)) {
    // AWQ layout and act-order: the MFMA kernel that unpacks the weights into LDS
    const MoeLaunch ml{mv, w->num_experts, tokens, pairs};
    return launch_gemm_awq(e0, x, nullptr, y, tokens, dtype, workspace, workspace_bytes, stream, &ml);
  } else {
    set_error("q4_moe_linear: no grouped kernel for tokens=%d K=%d N=%d groupsize=%d", tokens, e0->K, e0->N,
              e0->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_moe_linear: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host

using namespace q4host;

extern "C" {

int q4_moe_route_grouped(const void* gating, int gating_dtype, int tokens, int experts, int topk, int renormalize,
                         int num_expert_group, int topk_group, float* topk_weights, int32_t* topk_ids,
                         int32_t* sorted_tokens, int32_t* pair_slot, int32_t* expert_offsets, void* stream) {
  if (tokens < 0 || experts < 1 || experts > q4::kMoeMaxExperts || topk < 1 || topk > q4::kMoeMaxTopk ||
      topk > experts) {
    set_error("q4_moe_route: tokens=%d experts=%d (1..%d) topk=%d (1..%d, <= experts)", tokens, experts,
              q4::kMoeMaxExperts, topk, q4::kMoeMaxTopk);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (num_expert_group != 0 &&
      (num_expert_group < 1 || num_expert_group > 32 || experts % num_expert_group != 0 || topk_group < 1 ||
       topk_group > num_expert_group || topk > topk_group * (experts / num_expert_group))) {
    set_error("q4_moe_route: %d groups (1..32, dividing %d experts), %d of them kept, topk=%d must fit in them",
              num_expert_group, experts, topk_group, topk);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (expert_offsets == nullptr ||
      (tokens > 0 && (gating == nullptr || topk_weights == nullptr || topk_ids == nullptr ||
                      sorted_tokens == nullptr || pair_slot == nullptr))) {
    set_error("q4_moe_route: null pointer");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = (hipStream_t)stream;
  // one thread per token, one workgroup: a few tokens need a single wave
  const int threads = tokens >= 1024 ? 1024 : (tokens <= 64 ? 64 : ((tokens + 63) / 64) * 64);
  const dim3 grid(1), block((unsigned)threads);
  if (gating_dtype == Q4_DTYPE_F16)
    hipLaunchKernelGGL(q4::moe_route_kernel<Q4_DTYPE_F16>, grid, block, 0, s, gating, tokens, experts, topk,
                       renormalize, num_expert_group, topk_group, topk_weights, topk_ids, sorted_tokens, pair_slot,
                       expert_offsets);
  else if (gating_dtype == Q4_DTYPE_BF16)
    hipLaunchKernelGGL(q4::moe_route_kernel<Q4_DTYPE_BF16>, grid, block, 0, s, gating, tokens, experts, topk,
                       renormalize, num_expert_group, topk_group, topk_weights, topk_ids, sorted_tokens, pair_slot,
                       expert_offsets);
  else if (gating_dtype == Q4_DTYPE_F32)
    hipLaunchKernelGGL(q4::moe_route_kernel<Q4_DTYPE_F32>, grid, block, 0, s, gating, tokens, experts, topk,
                       renormalize, num_expert_group, topk_group, topk_weights, topk_ids, sorted_tokens, pair_slot,
                       expert_offsets);
  else {
    set_error("q4_moe_route: unknown gating dtype %d", gating_dtype);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_moe_route: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

int q4_moe_route(const void* gating, int gating_dtype, int tokens, int experts, int topk, int renormalize,
                 float* topk_weights, int32_t* topk_ids, int32_t* sorted_tokens, int32_t* pair_slot,
                 int32_t* expert_offsets, void* stream) {
  return q4_moe_route_grouped(gating, gating_dtype, tokens, experts, topk, renormalize, 0, 0, topk_weights, topk_ids,
                              sorted_tokens, pair_slot, expert_offsets, stream);
}

int q4_moe_linear(const q4_moe_weight* w, const void* x, const int32_t* x_rows, const int32_t* expert_offsets,
                  void* y, int tokens, int topk, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = validate_moe_weight(w, "q4_moe_linear");
  if (rc != Q4_OK) return rc;
  if (dtype != Q4_DTYPE_F16 && dtype != Q4_DTYPE_BF16) {
    set_error("q4_moe_linear: unknown dtype %d", dtype);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (tokens < 0 || topk < 1 || topk > q4::kMoeMaxTopk || (long)tokens * topk > 0x7fffffffL) {
    set_error("q4_moe_linear: tokens=%d topk=%d", tokens, topk);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (tokens == 0) return Q4_OK;
  if (x == nullptr || y == nullptr || expert_offsets == nullptr) {
    set_error("q4_moe_linear: null x / y / expert_offsets");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)workspace) & 15u) != 0) {
    set_error("q4_moe_linear: x, y and the workspace must be 16-byte aligned");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return launch_moe_linear(w, x, x_rows, expert_offsets, y, tokens, topk, dtype, workspace, workspace_bytes,
                           (hipStream_t)stream);
}

int q4_moe_linear_gate_up(const q4_moe_weight* w, const void* x, const int32_t* x_rows, const int32_t* expert_offsets,
                          void* y, int tokens, int topk, int dtype, int act, void* workspace, size_t workspace_bytes,
                          void* stream) {
  int rc = validate_moe_weight(w, "q4_moe_linear_gate_up");
  if (rc != Q4_OK) return rc;
  if ((dtype != Q4_DTYPE_F16 && dtype != Q4_DTYPE_BF16) || act < Q4_ACT_SILU || act > Q4_ACT_GELU) {
    set_error("q4_moe_linear_gate_up: dtype=%d act=%d", dtype, act);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (tokens < 0 || topk < 1 || topk > q4::kMoeMaxTopk || (long)tokens * topk > 0x7fffffffL || w->expert0.N % 16 != 0) {
    set_error("q4_moe_linear_gate_up: tokens=%d topk=%d N=%d", tokens, topk, w->expert0.N);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (tokens == 0) return Q4_OK;
  if (x == nullptr || y == nullptr || expert_offsets == nullptr) {
    set_error("q4_moe_linear_gate_up: null x / y / expert_offsets");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)workspace) & 15u) != 0) {
    set_error("q4_moe_linear_gate_up: x, y and the workspace must be 16-byte aligned");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return launch_moe_linear(w, x, x_rows, expert_offsets, y, tokens, topk, dtype, workspace, workspace_bytes,
                           (hipStream_t)stream, act + 1);
}

int q4_moe_combine(const void* y_sorted, const float* topk_weights, const int32_t* pair_slot, void* out, int tokens,
                   int topk, int N, int dtype, void* stream) {
  if (tokens < 0 || tokens > 65535 * 16 || topk < 1 || topk > q4::kMoeMaxTopk || N < 8 || N % 8 != 0 ||
      (dtype != Q4_DTYPE_F16 && dtype != Q4_DTYPE_BF16)) {
    set_error("q4_moe_combine: tokens=%d topk=%d N=%d (multiple of 8) dtype=%d", tokens, topk, N, dtype);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (tokens == 0) return Q4_OK;
  if (y_sorted == nullptr || topk_weights == nullptr || pair_slot == nullptr || out == nullptr) {
    set_error("q4_moe_combine: null pointer");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  hipStream_t s = (hipStream_t)stream;
  const int per_block = 256 * 8;
  // rows beyond the grid's y limit are taken in slices
  for (int t0 = 0; t0 < tokens; t0 += 65535) {
    const int nt = tokens - t0 < 65535 ? tokens - t0 : 65535;
    const dim3 grid((unsigned)((N + per_block - 1) / per_block), (unsigned)nt);
    const float* tw = topk_weights + (size_t)t0 * topk;
    const int32_t* ps = pair_slot + (size_t)t0 * topk;
    uint16_t* o = (uint16_t*)out + (size_t)t0 * N;
    if (dtype == Q4_DTYPE_F16)
      hipLaunchKernelGGL(q4::moe_combine_kernel<Q4_DTYPE_F16>, grid, dim3(256), 0, s, (const uint16_t*)y_sorted, tw, ps,
                         o, topk, N);
    else
      hipLaunchKernelGGL(q4::moe_combine_kernel<Q4_DTYPE_BF16>, grid, dim3(256), 0, s, (const uint16_t*)y_sorted, tw,
                         ps, o, topk, N);
  }
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_moe_combine: launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

size_t q4_moe_workspace_bytes(const q4_moe_weight* w, int tokens, int topk) {
  if (validate_moe_weight(w, "q4_moe_workspace_bytes") != Q4_OK || tokens < 0 || topk < 1) return 0;
  return moe_workspace_bytes(w, tokens, topk);
}

}  // extern "C"
