// C ABI of libq4linear.so: argument validation, path selection, error reporting.
// Nothing here allocates device memory or synchronises; every launch goes to the
// caller's stream.
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "q4_common.cuh"

namespace {
thread_local char g_error[512] = "";
}

namespace q4host {
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}
}  // namespace q4host

using namespace q4host;

static int validate_weight(const q4_weight* w, const char* who) {
  if (w == nullptr) {
    set_error("%s: null q4_weight", who);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (w->layout != Q4_LAYOUT_GPTQ && w->layout != Q4_LAYOUT_AWQ) {
    set_error("%s: unknown layout %d", who, w->layout);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (w->K < 0 || w->N < 0 || w->K % 8 != 0 || w->N % 8 != 0) {
    set_error("%s: K=%d and N=%d must be non-negative multiples of 8", who, w->K, w->N);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (w->K == 0 || w->N == 0) return Q4_OK;
  if (w->qweight == nullptr || w->qzeros == nullptr || w->scales == nullptr) {
    set_error("%s: null qweight/qzeros/scales", who);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  // the kernels fetch all tensors with 16-byte loads
  if ((((uintptr_t)w->qweight | (uintptr_t)w->qzeros | (uintptr_t)w->scales | (uintptr_t)w->g_idx) & 15u) != 0) {
    set_error("%s: qweight, qzeros, scales and g_idx must be 16-byte aligned", who);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (w->groupsize < 1 || w->num_groups < 1) {
    set_error("%s: groupsize=%d num_groups=%d must be positive", who, w->groupsize, w->num_groups);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (w->g_idx == nullptr && (long)w->num_groups * w->groupsize < w->K) {
    set_error("%s: %d groups of %d rows do not cover K=%d", who, w->num_groups, w->groupsize, w->K);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (w->layout == Q4_LAYOUT_AWQ && w->g_idx != nullptr) {
    set_error("%s: g_idx is not defined for the AWQ layout", who);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return Q4_OK;
}

static int validate_dtype(int dtype, const char* who) {
  if (dtype != Q4_DTYPE_F16 && dtype != Q4_DTYPE_BF16) {
    set_error("%s: unknown dtype %d", who, dtype);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return Q4_OK;
}

extern "C" {

int q4_abi_version(void) { return 1; }

const char* q4_last_error(void) { return g_error; }

int q4_dequant(const q4_weight* w, void* w_out, int dtype, void* stream) {
  int rc = validate_weight(w, "q4_dequant");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_dequant");
  if (rc != Q4_OK) return rc;
  if (w->K == 0 || w->N == 0) return Q4_OK;
  if (w_out == nullptr) {
    set_error("q4_dequant: null output");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (((uintptr_t)w_out & 15u) != 0) {
    set_error("q4_dequant: the output must be 16-byte aligned");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return launch_dequant(w, w_out, dtype, (hipStream_t)stream);
}

int q4_select_path(const q4_weight* w, int M, int dtype) {
  if (validate_weight(w, "q4_select_path") != Q4_OK) return Q4_ERR_INVALID_ARGUMENT;
  const bool contiguous_gptq = w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr;
  const long weights = (long)w->K * w->N;
  if (contiguous_gptq) {
    // Measured crossover on MI355X.  The decode kernel works in blocks of 16 rows that run side
    // by side (a second block costs little: the weights are shared through L2), the split-K
    // GEMM (64-row tiles up to M = 64) is nearly flat in M.  Decode / GEMM in us at M = 32:
    // 4096 x 4096 11.6 / 15.8, 4096 x 6144 12.7 / 17.3, 4096 x 14336 17.6 / 21.1, 8192 x 8192
    // 22.1 / 23.4, but 4096 x 28672 34.5 / 30.6, 8192 x 10240 38.4 / 32.6, 5120 x 13824 32.9 / 28.9,
    // 14336 x 4096 30.5 / 23.5 (at M = 17: 25.7 / 22.9).  From the third block on (M = 48) the
    // GEMM wins except on the smallest matrices (4096 x 4096: 12.6 / 17.9 at M = 64, 24.4 / 20.8
    // at M = 96; 2048 x 8192: 10.8 / 15.2 at M = 64).
    // Three and four blocks on the smallest matrices only while the decode launch stays one round
    // of workgroups (a slab that leaves room for one per CU and more workgroups than CUs: 5120 x 3072
    // at M = 48 20.4 / 14.7), four blocks only up to K = 4096 (M = 64: 5120 x 2560 21.2 / 15.1,
    // 8960 x 1536 22.6 / 15.4, 6912 x 2304 24.3 / 15.5, but 3072 x 5120 14.5 / 15.0, 2560 x 6144 12.8 / 15.2).
    bool blocks34 = M > 32 && M <= 64 && weights <= (1L << 24) && (M <= 48 || w->K <= 4096) && gemv_supported(w, M, dtype);
    if (blocks34) {
      const GemvConfig c = gemv_pick_config(w, M);
      const long mchunks = (M + c.rows_per_block - 1) / c.rows_per_block;
      const long wgs = (long)(w->N / (16 * c.words * c.wcol)) * mchunks * c.splits;
      const long chunks = w->K / 128;
      const long slab = (long)c.rows_per_block * ((chunks + c.splits - 1) / c.splits * 256 + 16);
      if (slab > 75 * 1024 && wgs > 256) blocks34 = false;
    }
    // Two blocks: up to K = 4096 (us at M = 32, decode / prefill: 4096 x 14336 18.7 / 19.3, 3072 x 16384
    // 15.1 / 17.2, but 6144 x 6144 23.5 / 17.0, 8192 x 7168 31.0 / 19.5, 8192 x 8192 22.5 / 20.3, 5120 x 5120
    // 21.3 / 15.2), beyond that on the smallest matrices only (5120 x 3072 12.1 / 13.6).
    const bool blocks2 = M <= 32 && weights <= (w->K <= 4096 ? (1L << 26) : (1L << 24));
    bool small = M <= 16 || gemv_rows32_supported(w, M) || blocks2 || blocks34;
    // bf16: past 16 rows the decode kernel converts every unpacked pair and the prefill kernel does
    // not; it keeps 17 to 32 rows on the smallest matrices only (us at M = 24, decode / prefill:
    // 4096 x 4096 12.7 / 13.8, but 4096 x 14336 23.4 / 19.0, 2048 x 8192 13.4 / 11.7, 8192 x 8192 at
    // M = 17 20.9 / 18.8, 14336 x 4096 at M = 20 20.4 / 19.0)
    if (dtype == Q4_DTYPE_BF16 && M > 16) small = M <= 32 && weights <= (1L << 24) && w->K >= 3072;
    if (small && gemv_supported(w, M, dtype)) return Q4_PATH_GEMV;
    if (gemm_supported(w, M, dtype)) return Q4_PATH_GEMM;
    if (gemv_supported(w, M, dtype)) return Q4_PATH_GEMV;
    return Q4_PATH_GENERIC;
  }
  // AWQ and act-order: the decode kernels take any M in row chunks of 16; the MFMA kernel
  // that unpacks the weights into LDS (split-K when its tile grid is small) takes over where
  // it measured faster on MI355X.
  // Act-order: from M = 33 on when its parameter table fits in LDS (two 16-row blocks of the
  // decode kernel, which is flat in M within a block, against the MFMA kernel, flat in M up to
  // 128 rows, us at M = 32: 4096 x 4096 14.2 / 20.3, 14336 x 4096 27.0 / 43.4, 8192 x 10240
  // 41.6 / 56.4, 28672 x 8192 92.7 / 153; at M = 48 the three blocks win on some shapes, 18.5 /
  // 21.3 and 45.8 / 55.5, and lose on others, 46.6 / 42.7 and 182 / 155), from about M = 48 on
  // when it has to gather scales and zero points from global memory (~2x slower per tile).
  // AWQ: up to 6 rows the decode kernel that feeds the words to the MFMA as stored; from 7 rows on
  // the MFMA kernel that unpacks them in registers wherever it applies (split-K on small tile
  // grids, flat in M up to 32 rows: 17.4 against 28.3 us for 4096 x 14336 at M = 16, 17.9 against
  // 31.4 us for 14336 x 4096, 12.5 against 12.7 us for 4096 x 4096).  Other AWQ weights (N not a
  // multiple of 256, groups shorter than 64 rows): the general decode kernel, whose time grows
  // with every row, up to the M at which the kernel that unpacks through LDS measured faster:
  // 4096 x 4096 9, 4096 x 6144 14, 5120 x 5120 16, 11008 x 4096 10; above 16 for the larger
  // layers; 28672 x 8192 and 8192 x 28672 up to 32 rows.
  bool small = M <= 16 || (w->layout == Q4_LAYOUT_GPTQ && (M <= 32 || (M <= 48 && !gemm_act_order_table(w))));
  if (w->layout == Q4_LAYOUT_AWQ) {
    int first_gemm_m = 17;
    if (weights >= (1L << 27)) first_gemm_m = 33;
    else if (weights <= (1L << 24)) first_gemm_m = 9;
    else if (weights <= (1L << 25)) first_gemm_m = 14;
    else if ((w->K / 128) % 8 != 0 && weights <= (1L << 26)) first_gemm_m = 10;
    // (the words-as-stored decode kernel takes a second accumulator set from five rows on; since
    // its K splits meet in the fixed-point cells at any row count it holds five and six rows --
    // decode / this kernel in us at M = 6: 14336 x 4096 16.8 / 19.8, 4096 x 4096 11.3 / 13.5,
    // 4096 x 6144 11.6 / 13.7, 4096 x 28672 23.2 / 23.5, 4096 x 14336 16.4 / 15.6 -- and loses from
    // eight on: 14.9 / 13.5, 15.0 / 13.8, 17.0 / 16.0, except 14336 x 4096 17.4 / 20.0)
    if (gemm_awq_direct_supported(w, M, dtype)) first_gemm_m = 7;
    small = M < first_gemm_m;
  }
  if (!small && gemm_awq_supported(w, M, dtype)) return Q4_PATH_GEMM;
  if (gemv_supported(w, M, dtype)) return Q4_PATH_GEMV;
  // (what the decode kernels do not take, e.g. an act-order table too large for LDS: the MFMA kernel takes any M)
  if (gemm_awq_supported(w, M, dtype)) return Q4_PATH_GEMM;
  return Q4_PATH_GENERIC;
}

// Bytes of split-K partial sums the decode kernels would write for this weight at M rows:
// the launcher's own decomposition, for the plain call and (where it exists) the gated-MLP one.
static size_t decode_partial_bytes(const q4_weight* w, int M) {
  if (!gemv_supported(w, M, Q4_DTYPE_F16) && !gemv_supported(w, M, Q4_DTYPE_BF16)) return 0;
  int splits = gemv_pick_config(w, M).splits;
  if (w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr && w->N % 128 == 0) {
    const int s = gemv_pick_config(w, M, true).splits;
    if (s > splits) splits = s;
  }
  return splits > 1 ? (size_t)splits * M * w->N * sizeof(float) : 0;
}

size_t q4_workspace_bytes_for(const q4_weight* w, int M) {
  if (validate_weight(w, "q4_workspace_bytes_for") != Q4_OK || M < 1 || w->K == 0 || w->N == 0)
    return Q4_WORKSPACE_COUNTER_BYTES;
  const size_t decode = decode_partial_bytes(w, M);
  const size_t prefill = gemm_workspace_bytes(M, w->K, w->N);
  return (size_t)Q4_WORKSPACE_COUNTER_BYTES + (decode > prefill ? decode : prefill);
}

int q4_linear_plan(const q4_weight* w, int M, int dtype, int* path, size_t* workspace_bytes) {
  int rc = validate_weight(w, "q4_linear_plan");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_linear_plan");
  if (rc != Q4_OK) return rc;
  if (M < 0 || path == nullptr || workspace_bytes == nullptr) {
    set_error("q4_linear_plan: negative M=%d or null output pointer", M);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  *path = (M == 0 || w->K == 0 || w->N == 0) ? Q4_PATH_GENERIC : q4_select_path(w, M, dtype);
  *workspace_bytes = q4_workspace_bytes_for(w, M);
  return Q4_OK;
}

size_t q4_workspace_bytes(int M, int K, int N) {
  if (M < 1 || K < 1 || N < 1) return Q4_WORKSPACE_COUNTER_BYTES;
  // Upper bound over the three decode kernels (their column tiles and split choices differ)
  // for every weight of this shape: the act-order kernel's choice also depends on the number
  // of groups (its parameter table shares LDS with the activation slab), so it is bounded over
  // the group sizes 32 .. 1024 and "one group".
  size_t decode = 0;
  if (K % 128 == 0 && N % 64 == 0) {
    static const int32_t fake_idx = 0;
    q4_weight w = {};
    w.K = K;
    w.N = N;
    const int m_lo = M <= 16 ? 1 : M, m_hi = M;
    for (int variant = 0; variant < 3; ++variant) {
      w.layout = variant == 1 ? Q4_LAYOUT_AWQ : Q4_LAYOUT_GPTQ;
      w.g_idx = variant == 2 ? &fake_idx : nullptr;  // only tested against NULL
      if (variant == 1 && N % 256 != 0) continue;
      static const int kGroupSizes[] = {128, 32, 64, 256, 512, 1024, 1 << 30};
      for (int gs : kGroupSizes) {
        // the AWQ kernel does not look at the group count; contiguous GPTQ groups shorter than a
        // chunk run on a different kernel, with its own decomposition
        if (gs != 128 && (variant == 1 || (variant == 0 && gs != 32))) continue;
        if (gs < K && K % gs != 0) continue;
        w.groupsize = gs < K ? gs : K;
        w.num_groups = K / w.groupsize;
        for (int m = m_lo; m <= m_hi; ++m) {
          const size_t b = decode_partial_bytes(&w, m) / m * M;
          if (b > decode) decode = b;
        }
      }
    }
  }
  // decode: split-K partial sums; prefill: split-K partial tiles of under-filled GEMM grids
  const size_t prefill = gemm_workspace_bytes(M, K, N);
  return (size_t)Q4_WORKSPACE_COUNTER_BYTES + (decode > prefill ? decode : prefill);
}

int q4_linear_ex(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                 void* workspace, size_t workspace_bytes, int path, void* stream) {
  int rc = validate_weight(w, "q4_linear");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_linear");
  if (rc != Q4_OK) return rc;
  if (M < 0) {
    set_error("q4_linear: negative M=%d", M);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || w->N == 0) return Q4_OK;
  if (y == nullptr || (x == nullptr && w->K > 0)) {
    set_error("q4_linear: null x or y");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if ((((uintptr_t)x | (uintptr_t)y | (uintptr_t)workspace) & 15u) != 0 || ((uintptr_t)bias & 1u) != 0) {
    set_error("q4_linear: x, y and the workspace must be 16-byte aligned (bias: 2-byte)");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (path == Q4_PATH_AUTO) path = q4_select_path(w, M, dtype);
  switch (path) {
    case Q4_PATH_GEMV:
      return launch_gemv(w, x, bias, y, M, dtype, workspace, workspace_bytes, nullptr,
                         (hipStream_t)stream);
    case Q4_PATH_GEMM:
      if (w->layout == Q4_LAYOUT_AWQ || w->g_idx != nullptr)
        return launch_gemm_awq(w, x, bias, y, M, dtype, workspace, workspace_bytes, (hipStream_t)stream);
      return launch_gemm(w, x, bias, y, M, dtype, workspace, workspace_bytes, (hipStream_t)stream);
    case Q4_PATH_GENERIC:
      return launch_generic(w, x, bias, y, M, dtype, (hipStream_t)stream);
    default:
      set_error("q4_linear: unknown path %d", path);
      return Q4_ERR_INVALID_ARGUMENT;
  }
}

int q4_gptq_solve_block(float* W, const float* U, float* Q, float* err, float* loss, float* scale, float* zero,
                        int rows, int K, int i1, int count, int groupsize, int num_groups, int sym, void* stream) {
  if (W == nullptr || U == nullptr || Q == nullptr || err == nullptr || loss == nullptr || scale == nullptr ||
      zero == nullptr) {
    set_error("q4_gptq_solve_block: null pointer");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (rows < 1 || K < 1 || i1 < 0 || count < 1 || count > 128 || i1 + count > K) {
    set_error("q4_gptq_solve_block: bad rows=%d, K=%d or block [%d, %d) (at most 128 columns)", rows, K, i1,
              i1 + count);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (groupsize > 0 ? (long)num_groups * groupsize < K : num_groups != 1) {
    set_error("q4_gptq_solve_block: %d groups of %d columns do not cover K=%d", num_groups, groupsize, K);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return launch_gptq_solve_block(W, U, Q, err, loss, scale, zero, rows, K, i1, count, groupsize, num_groups, sym,
                                 (hipStream_t)stream);
}

int q4_moe_gather_columns(const void* x, const int32_t* x_rows, const int32_t* expert_offsets, const int32_t* perms,
                          void* out, int num_experts, int pairs, int K, void* stream) {
  if (num_experts < 1 || pairs < 0 || K < 0) {
    set_error("q4_moe_gather_columns: bad num_experts=%d, pairs=%d or K=%d", num_experts, pairs, K);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (pairs == 0 || K == 0) return Q4_OK;
  if (x == nullptr || expert_offsets == nullptr || perms == nullptr || out == nullptr || x == out) {
    set_error("q4_moe_gather_columns: null pointer, or output aliasing the input");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (K % 8 != 0) {
    set_error("q4_moe_gather_columns: K=%d must be a multiple of 8", K);
    return Q4_ERR_UNSUPPORTED;
  }
  return launch_moe_gather_columns(x, x_rows, expert_offsets, perms, out, num_experts, pairs, K, (hipStream_t)stream);
}

static size_t perm_gather_offset(int M, int K, int N) {
  return (q4_workspace_bytes(M, K, N) + 255) & ~(size_t)255;
}

size_t q4_workspace_bytes_perm(int M, int K, int N) {
  if (M < 1 || K < 1 || N < 1) return q4_workspace_bytes(M, K, N);
  return perm_gather_offset(M, K, N) + (size_t)M * K * 2;
}

int q4_linear_perm(const q4_weight* w, const int32_t* perm, const void* x, const void* bias, void* y, int M,
                   int dtype, void* workspace, size_t workspace_bytes, int path, void* stream) {
  if (perm == nullptr) return q4_linear_ex(w, x, bias, y, M, dtype, workspace, workspace_bytes, path, stream);
  int rc = validate_weight(w, "q4_linear_perm");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_linear_perm");
  if (rc != Q4_OK) return rc;
  if (w->layout != Q4_LAYOUT_GPTQ || w->g_idx != nullptr) {
    set_error("q4_linear_perm: the weight must be a GPTQ matrix whose rows are in group order (g_idx NULL)");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M < 0) {
    set_error("q4_linear_perm: negative M=%d", M);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || w->N == 0) return Q4_OK;
  if (y == nullptr || x == nullptr) {
    set_error("q4_linear_perm: null x or y");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if ((((uintptr_t)x | (uintptr_t)y) & 15u) != 0 || ((uintptr_t)bias & 1u) != 0) {
    set_error("q4_linear_perm: x and y must be 16-byte aligned (bias: 2-byte)");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (path == Q4_PATH_AUTO) path = q4_select_path(w, M, dtype);
  // Decode of a few rows with a short K: the kernel reads x through perm while it stages its
  // activation slab.  Every workgroup gathers its own copy, so the saved launch (~2.5 us) is
  // soon outweighed: measured against the separate pass at M = 1, 4096 x 4096 6.4 / 7.8 us,
  // 4096 x 28672 15.8 / 17.3, but 14336 x 4096 13.4 / 12.3, 28672 x 8192 29.0 / 26.0; at M = 4
  // 4096 x 4096 9.1 / 10.6, 4096 x 6144 9.8 / 10.7, but 4096 x 28672 20.2 / 19.2; at M = 8
  // 4096 x 6144 12.7 / 11.7; at M = 16 4096 x 6144 18.1 / 14.3, 14336 x 4096 37.9 / 20.0.
  if (path == Q4_PATH_GEMV && w->K <= 4096 && (M <= 2 || (M <= 4 && w->N <= 8192)))
    return launch_gemv(w, x, bias, y, M, dtype, workspace, workspace_bytes, nullptr, (hipStream_t)stream, 0, perm);
  // otherwise one gather pass into the tail of the workspace, then the kernel of the plain call
  if (w->K % 8 != 0) {
    set_error("q4_linear_perm: K=%d must be a multiple of 8", w->K);
    return Q4_ERR_UNSUPPORTED;
  }
  const size_t offset = perm_gather_offset(M, w->K, w->N);
  const size_t need = offset + (size_t)M * w->K * 2;
  if (workspace == nullptr || workspace_bytes < need) {
    set_error("q4_linear_perm: workspace of %zu bytes needed (q4_workspace_bytes_perm), %zu given", need,
              workspace_bytes);
    return Q4_ERR_WORKSPACE;
  }
  void* x_seq = (char*)workspace + offset;
  rc = launch_gather_columns(x, perm, x_seq, M, w->K, (hipStream_t)stream);
  if (rc != Q4_OK) return rc;
  return q4_linear_ex(w, x_seq, bias, y, M, dtype, workspace, offset, path, stream);
}

int q4_linear_gate_up_perm(const q4_weight* w, const int32_t* perm, const void* x, const void* bias, void* y, int M,
                           int dtype, int act, void* workspace, size_t workspace_bytes, void* stream) {
  if (perm == nullptr) return q4_linear_gate_up(w, x, bias, y, M, dtype, act, workspace, workspace_bytes, stream);
  int rc = validate_weight(w, "q4_linear_gate_up_perm");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_linear_gate_up_perm");
  if (rc != Q4_OK) return rc;
  if (act != Q4_ACT_SILU && act != Q4_ACT_GELU_TANH && act != Q4_ACT_GELU) {
    set_error("q4_linear_gate_up_perm: unknown activation %d", act);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M < 0 || (w->N & 1) || w->layout != Q4_LAYOUT_GPTQ || w->g_idx != nullptr) {
    set_error("q4_linear_gate_up_perm: bad M=%d, odd N=%d, or a weight that is not a GPTQ matrix in group order", M,
              w->N);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || w->N == 0) return Q4_OK;
  if (y == nullptr || x == nullptr) {
    set_error("q4_linear_gate_up_perm: null x or y");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if ((((uintptr_t)x | (uintptr_t)y) & 15u) != 0 || ((uintptr_t)bias & 1u) != 0) {
    set_error("q4_linear_gate_up_perm: x and y must be 16-byte aligned (bias: 2-byte)");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (q4_select_path(w, M, dtype) == Q4_PATH_GEMM && gemm_gate_up_supported(w, M, dtype)) {
    // prefill: gather the activation columns into the workspace tail, then the fused MFMA kernel
    const size_t offset = perm_gather_offset(M, w->K, w->N);
    const size_t need = offset + (size_t)M * w->K * 2;
    if (workspace == nullptr || workspace_bytes < need || w->K % 8 != 0) {
      set_error("q4_linear_gate_up_perm: workspace of %zu bytes needed (q4_workspace_bytes_perm), %zu given", need,
                workspace_bytes);
      return Q4_ERR_WORKSPACE;
    }
    void* x_seq = (char*)workspace + offset;
    rc = launch_gather_columns(x, perm, x_seq, M, w->K, (hipStream_t)stream);
    if (rc != Q4_OK) return rc;
    return launch_gemm_gate_up(w, x_seq, bias, y, M, dtype, act, (hipStream_t)stream);
  }
  if (!(q4_select_path(w, M, dtype) == Q4_PATH_GEMV && gemv_gate_up_supported(w, M, dtype))) {
    set_error("q4_linear_gate_up_perm: no fused kernel for this problem (M=%d K=%d N=%d groupsize=%d)", M, w->K, w->N,
              w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  // the fused kernel runs for one or two rows: with a short K it gathers while staging (see q4_linear_perm)
  if (w->K <= 4096)
    return launch_gemv(w, x, bias, y, M, dtype, workspace, workspace_bytes, nullptr, (hipStream_t)stream, act + 1, perm);
  const size_t offset = perm_gather_offset(M, w->K, w->N);
  const size_t need = offset + (size_t)M * w->K * 2;
  if (workspace == nullptr || workspace_bytes < need || w->K % 8 != 0) {
    set_error("q4_linear_gate_up_perm: workspace of %zu bytes needed (q4_workspace_bytes_perm), %zu given", need,
              workspace_bytes);
    return Q4_ERR_WORKSPACE;
  }
  void* x_seq = (char*)workspace + offset;
  rc = launch_gather_columns(x, perm, x_seq, M, w->K, (hipStream_t)stream);
  if (rc != Q4_OK) return rc;
  return launch_gemv(w, x_seq, bias, y, M, dtype, workspace, offset, nullptr, (hipStream_t)stream, act + 1);
}

int q4_linear_gate_up(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                      int act, void* workspace, size_t workspace_bytes, void* stream) {
  int rc = validate_weight(w, "q4_linear_gate_up");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_linear_gate_up");
  if (rc != Q4_OK) return rc;
  if (act != Q4_ACT_SILU && act != Q4_ACT_GELU_TANH && act != Q4_ACT_GELU) {
    set_error("q4_linear_gate_up: unknown activation %d", act);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M < 0 || (w->N & 1)) {
    set_error("q4_linear_gate_up: bad M=%d or odd N=%d", M, w->N);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || w->N == 0) return Q4_OK;
  if (y == nullptr || (x == nullptr && w->K > 0)) {
    set_error("q4_linear_gate_up: null x or y");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if ((((uintptr_t)x | (uintptr_t)y) & 15u) != 0 || ((uintptr_t)bias & 1u) != 0) {
    set_error("q4_linear_gate_up: x and y must be 16-byte aligned (bias: 2-byte)");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  // Decode: the kernels with eight words per lane.  Prefill: the MFMA kernel with a lane's two
  // columns set to (gate c, up c), where it runs unsplit.
  const int path = q4_select_path(w, M, dtype);
  if (path == Q4_PATH_GEMV && gemv_gate_up_supported(w, M, dtype))
    return launch_gemv(w, x, bias, y, M, dtype, workspace, workspace_bytes, nullptr, (hipStream_t)stream, act + 1);
  if (path == Q4_PATH_GEMM && gemm_gate_up_supported(w, M, dtype))
    return launch_gemm_gate_up(w, x, bias, y, M, dtype, act, (hipStream_t)stream);
  set_error("q4_linear_gate_up: no fused kernel for this problem (layout=%d g_idx=%p M=%d K=%d N=%d groupsize=%d)",
            w->layout, (const void*)w->g_idx, M, w->K, w->N, w->groupsize);
  return Q4_ERR_UNSUPPORTED;
}

int q4_linear_gate_up_plan(const q4_weight* w, int M, int dtype, int* fused) {
  int rc = validate_weight(w, "q4_linear_gate_up_plan");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_linear_gate_up_plan");
  if (rc != Q4_OK) return rc;
  if (fused == nullptr || M < 0) {
    set_error("q4_linear_gate_up_plan: null output or negative M=%d", M);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  *fused = 0;
  if (M == 0 || w->K == 0 || w->N == 0 || (w->N & 1)) return Q4_OK;
  const int path = q4_select_path(w, M, dtype);
  if (path == Q4_PATH_GEMM) {
    *fused = gemm_gate_up_supported(w, M, dtype) ? 1 : 0;
    return Q4_OK;
  }
  if (path != Q4_PATH_GEMV || !gemv_gate_up_supported(w, M, dtype)) return Q4_OK;
  // One or two rows on a large layer: the plain call runs the lean / short-launch kernels there,
  // and that followed by the elementwise kernel beats the decode kernel with the gated epilogue
  // (us on MI355X, fused / two launches: 4096 x 28672 17.7 / 16.6 at M = 1, 3072 x 16384 17.1 / 11.3 at
  // M = 2, 8192 x 57344 53.7 / 47.5 at M = 2; 4096 x 22016 at M = 1, 16.1 / 17.0, is the one shape
  // measured that loses).  Smaller layers keep the single launch.
  const bool large = gemv_lean_supported(w, dtype) && (long)w->K * w->N >= (1L << 25) && w->K >= 1024;
  *fused = large ? 0 : 1;
  return Q4_OK;
}

int q4_act_mul(const void* gate_up, void* y, int M, int inter, int dtype, int act, void* stream) {
  int rc = validate_dtype(dtype, "q4_act_mul");
  if (rc != Q4_OK) return rc;
  if (act != Q4_ACT_SILU && act != Q4_ACT_GELU_TANH && act != Q4_ACT_GELU) {
    set_error("q4_act_mul: unknown activation %d", act);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M < 0 || inter < 0) {
    set_error("q4_act_mul: negative M=%d or intermediate size %d", M, inter);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || inter == 0) return Q4_OK;
  if (gate_up == nullptr || y == nullptr) {
    set_error("q4_act_mul: null pointer");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return launch_act_mul(gate_up, y, M, inter, dtype, act, (hipStream_t)stream);
}

int q4_gptq_make_sequential(const uint32_t* qweight, const int32_t* perm, uint32_t* qweight_out, int K, int N,
                            void* stream) {
  if (qweight == nullptr || perm == nullptr || qweight_out == nullptr || qweight == qweight_out) {
    set_error("q4_gptq_make_sequential: null pointer, or output aliasing the input");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (K < 8 || K % 8 != 0 || N < 1) {
    set_error("q4_gptq_make_sequential: K=%d must be a positive multiple of 8, N=%d positive", K, N);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (K / 8 > 65535) {
    set_error("q4_gptq_make_sequential: K=%d has more than 65535 packed rows", K);
    return Q4_ERR_UNSUPPORTED;
  }
  return launch_make_sequential(qweight, perm, qweight_out, K, N, (hipStream_t)stream);
}

int q4_gather_columns(const void* x, const int32_t* perm, void* out, int M, int K, void* stream) {
  if (M < 0 || K < 0) {
    set_error("q4_gather_columns: negative M=%d or K=%d", M, K);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || K == 0) return Q4_OK;
  if (x == nullptr || perm == nullptr || out == nullptr || x == out) {
    set_error("q4_gather_columns: null pointer, or output aliasing the input");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (K % 8 != 0) {
    set_error("q4_gather_columns: K=%d must be a multiple of 8", K);
    return Q4_ERR_UNSUPPORTED;
  }
  return launch_gather_columns(x, perm, out, M, K, (hipStream_t)stream);
}

// ---- q4_linear without a caller-provided workspace -------------------------------------
// The scratch memory of the split-K paths (tickets, accumulation cells, fp32 partial sums) lives
// in a file-scope device array instead of a caller's buffer.  In host code the array's name
// is only a stand-in for the symbol: its device address is looked up once per device.
#define Q4_SCRATCH_BYTES Q4_NOALLOC_SCRATCH_BYTES
static __device__ __align__(256) unsigned char scratch[Q4_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices] = {};
std::mutex g_scratch_mutex;

// Device address of `scratch` on the current device (looked up on first use), or nullptr with
// the error set.
void* scratch_of_current_device(const char* who) {
  int dev = -1;
  hipError_t err = hipGetDevice(&dev);
  if (err != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    set_error("%s: cannot identify the current device (%s, device %d)", who,
              err != hipSuccess ? hipGetErrorString(err) : "out of range", dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    err = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (err != hipSuccess || ptr == nullptr) {
      set_error("%s: hipGetSymbolAddress(scratch) failed on device %d: %s", who, dev, hipGetErrorString(err));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}
}  // namespace

int q4_noalloc_init(void) { return scratch_of_current_device("q4_noalloc_init") != nullptr ? Q4_OK : Q4_ERR_LAUNCH; }

int q4_linear_noalloc(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype, void* stream) {
  int rc = validate_weight(w, "q4_linear_noalloc");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_linear_noalloc");
  if (rc != Q4_OK) return rc;
  if (M < 0) {
    set_error("q4_linear_noalloc: negative M=%d", M);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M == 0 || w->N == 0) return Q4_OK;
  const int path = q4_select_path(w, M, dtype);
  // the decode kernels need their whole workspace; the prefill kernels fall back to unsplit
  // tiles when the partial tiles do not fit, so they run with whatever the array holds
  const size_t need = path == Q4_PATH_GEMV ? (size_t)Q4_WORKSPACE_COUNTER_BYTES + decode_partial_bytes(w, M)
                                           : (size_t)Q4_WORKSPACE_COUNTER_BYTES;
  if (need > Q4_SCRATCH_BYTES) {
    set_error("q4_linear_noalloc: M=%d K=%d N=%d needs %zu bytes of scratch, the built-in array holds %zu "
              "(use q4_linear with a workspace of q4_workspace_bytes_for())", M, w->K, w->N, need,
              (size_t)Q4_SCRATCH_BYTES);
    return Q4_ERR_WORKSPACE;
  }
  void* ptr = scratch_of_current_device("q4_linear_noalloc");
  if (ptr == nullptr) return Q4_ERR_LAUNCH;
  return q4_linear_ex(w, x, bias, y, M, dtype, ptr, Q4_SCRATCH_BYTES, path, stream);
}

int q4_linear(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
              void* workspace, size_t workspace_bytes, void* stream) {
  return q4_linear_ex(w, x, bias, y, M, dtype, workspace, workspace_bytes, Q4_PATH_AUTO, stream);
}

int q4_gemv_candidates(const q4_weight* w, int M, int dtype, int32_t* configs, int max_configs) {
  if (validate_weight(w, "q4_gemv_candidates") != Q4_OK || validate_dtype(dtype, "q4_gemv_candidates") != Q4_OK) return Q4_ERR_INVALID_ARGUMENT;
  if (configs == nullptr || max_configs < 0) {
    set_error("q4_gemv_candidates: null output");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (M < 1 || w->K == 0 || w->N == 0 || q4_select_path(w, M, dtype) != Q4_PATH_GEMV) return 0;
  if (w->layout == Q4_LAYOUT_AWQ) {
    // the words-as-stored kernel (up to 8 rows, 256-column wave tiles): K waves x K splits that
    // deal K evenly, between one and thirty-two waves per CU
    if (M > 8 || w->N % 256 != 0 || w->K % 128 != 0) return 0;
    const int achunks = w->K / 128;
    const long atiles = w->N / 256;
    static const int kAwqWaves[] = {8, 4, 2};
    static const int kAwqSplits[] = {1, 2, 4, 8, 7, 14, 3, 5, 6, 10, 12, 16};
    int na = 0;
    for (int wk : kAwqWaves) {
      for (int sp : kAwqSplits) {
        if (na >= max_configs) return na;
        if (wk * sp > achunks || achunks % (wk * sp) != 0) continue;
        const long waves = atiles * wk * sp;
        if (waves < 256 || waves > 8192) continue;
        configs[4 * na + 0] = 1;
        configs[4 * na + 1] = wk;
        configs[4 * na + 2] = sp;
        configs[4 * na + 3] = 0;
        ++na;
      }
    }
    return na;
  }
  // The short-launch kernel's decompositions: K waves per workgroup x workgroups along K.  Kept:
  // even K deals where the chunk count has them, between one and sixty-four waves per CU in all.
  const int chunks = w->K / 128;
  const long tiles = w->N / 64;
  static const int kWaves[] = {4, 8, 2, 1};
  static const int kSplits[] = {1, 2, 4, 8, 7, 14, 3, 5, 6, 10, 12, 16};
  int n = 0;
  for (int pass = 0; pass < 2 && n == 0; ++pass) {  // second pass: ragged deals, for a K without even ones
    for (int wk : kWaves) {
      for (int sp : kSplits) {
        if (n >= max_configs) return n;
        if (!gemv_direct_supported(w, M, dtype, wk, sp)) continue;
        if (pass == 0 && chunks % (wk * sp) != 0) continue;
        const long waves = tiles * wk * sp;
        if (waves < 256 || waves > 16384) continue;
        configs[4 * n + 0] = 1;
        configs[4 * n + 1] = wk;
        configs[4 * n + 2] = sp;
        configs[4 * n + 3] = -1;
        ++n;
      }
    }
  }
  return n;
}

size_t q4_gemv_tuned_workspace_bytes(const q4_weight* w, int M, int dtype, int wcol, int wk, int splits, int words) {
  (void)wcol;
  (void)wk;
  if (validate_weight(w, "q4_gemv_tuned_workspace_bytes") != Q4_OK || M < 1) return Q4_WORKSPACE_COUNTER_BYTES;
  if (words == -1) {
    const size_t need = gemv_direct_workspace_bytes(w, M, dtype, splits);
    return need > (size_t)Q4_WORKSPACE_COUNTER_BYTES ? need : (size_t)Q4_WORKSPACE_COUNTER_BYTES;
  }
  return (size_t)Q4_WORKSPACE_COUNTER_BYTES + (splits > 1 ? (size_t)splits * M * w->N * sizeof(float) : 0);
}

int q4_gemv_tuned(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                  void* workspace, size_t workspace_bytes, int wcol, int wk, int splits, int words,
                  void* stream) {
  int rc = validate_weight(w, "q4_gemv_tuned");
  if (rc == Q4_OK) rc = validate_dtype(dtype, "q4_gemv_tuned");
  if (rc != Q4_OK) return rc;
  if (M < 1 || x == nullptr || y == nullptr) {
    set_error("q4_gemv_tuned: bad M=%d or null x/y", M);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (words == -1)  // the short-launch kernel: wk K waves per workgroup, `splits` workgroups along K (wcol unused)
    return launch_gemv_direct(w, x, bias, y, M, dtype, workspace, workspace_bytes, wk, splits, (hipStream_t)stream);
  GemvConfig cfg{wcol, wk, splits, words};
  if (words == 0) {  // the lean contiguous-group kernel / the AWQ kernel that feeds the words as stored
    cfg.words = 4;
    cfg.lean = 1;
  } else if (words == 4 && gemv_rows32_kernel(w, M)) cfg.rows_per_block = 32;  // one workgroup for all rows
  return launch_gemv(w, x, bias, y, M, dtype, workspace, workspace_bytes, &cfg, (hipStream_t)stream);
}

}  // extern "C"
