/*
 * q4_linear.h -- C ABI of libq4linear.so: int4 weight-only quantized linear layer
 * (GPTQ and AWQ checkpoint layouts) for AMD MI355X (gfx950).
 *
 * The library is stateless: every buffer is owned by the caller (PyTorch tensors on
 * the Python side), nothing is allocated on the device, every call is asynchronous
 * on the HIP stream it is given and can be recorded into a HIP graph.  Functions
 * return 0 on success or a negative Q4_ERR_* code; q4_last_error() then describes
 * the failure (thread-local).  No C++ exception crosses this boundary.
 *
 * Tensor conventions (K = in-features, N = out-features, G = number of groups):
 *   GPTQ (layout 0): qweight int32 [K/8, N]  nibble j of word [r, n] = q[8r+j, n]
 *                    qzeros  int32 [G, N/8]  nibble j of word [g, c] = zstored[g, 8c+j]
 *                    effective zero = (zstored + 1) & 15
 *   AWQ  (layout 1): qweight int32 [K, N/8]  nibble p of word [k, c] = q[k, 8c+ORDER[p]]
 *                    qzeros  int32 [G, N/8]  same column order, used as stored
 *                    ORDER = {0, 2, 4, 6, 1, 3, 5, 7}
 *   scales fp16 [G, N] (always fp16, also for bf16 activations)
 *   g_idx  int32 [K] or NULL: group of row k (GPTQ act-order); NULL -> k / groupsize
 *   W[k, n] = round_to_dtype( float(scales[g(k), n]) * (q[k, n] - zero[g(k), n]) )
 *   y[m, n] = sum_k x[m, k] * W[k, n]  accumulated in fp32 (+ bias[n]), cast to dtype
 *   x [M, K], y [M, N], bias [N] (nullable) row-major contiguous in `dtype`.
 */
#ifndef Q4_LINEAR_H
#define Q4_LINEAR_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define Q4_LAYOUT_GPTQ 0
#define Q4_LAYOUT_AWQ 1

#define Q4_DTYPE_F16 0
#define Q4_DTYPE_BF16 1

#define Q4_OK 0
#define Q4_ERR_INVALID_ARGUMENT (-1) /* null pointer, bad enum, bad shape */
#define Q4_ERR_UNSUPPORTED (-2)      /* a shape the kernels do not cover */
#define Q4_ERR_WORKSPACE (-3)        /* workspace missing or too small */
#define Q4_ERR_LAUNCH (-4)           /* HIP reported a launch error */

/* Which kernel q4_linear picks; also accepted by q4_linear_ex to force one. */
#define Q4_PATH_AUTO 0
#define Q4_PATH_GEMV 1    /* split-K dequant GEMV, decode (small M) */
#define Q4_PATH_GEMM 2    /* dequant-to-LDS + MFMA GEMM, prefill (large M) */
#define Q4_PATH_GENERIC 3 /* shape-agnostic kernel for unaligned K / N */

/* Problem description shared by every entry point.  All device pointers handed to this library
 * (the four tensors below, activations, outputs, workspaces) must be 16-byte aligned, a bias
 * 2-byte aligned: the kernels fetch with 16-byte loads, and the entry points refuse anything
 * else with Q4_ERR_INVALID_ARGUMENT. */
typedef struct q4_weight {
  const uint32_t* qweight; /* packed nibbles, see layout above */
  const uint32_t* qzeros;  /* packed zero points [G, N/8] */
  const void* scales;      /* fp16 [G, N] */
  const int32_t* g_idx;    /* int32 [K] or NULL */
  int32_t K;               /* in-features, multiple of 8 */
  int32_t N;               /* out-features, multiple of 8 */
  int32_t groupsize;       /* rows per group when g_idx is NULL (K for "one group") */
  int32_t num_groups;      /* G: rows of scales / qzeros */
  int32_t layout;          /* Q4_LAYOUT_* */
} q4_weight;

/*
 * Materialise the dense dequantized weight W [K, N] in `dtype` (bit-exact with the
 * reference's dequantize step).  Replaces exllamav2 reconstruct_gptq_kernel
 * (server/exllamav2_kernels/exllamav2_kernels/cuda/q_matrix.cu:182-299, pybind
 * `reconstruct` path of ext.cpp) and exllama v1 reconstruct_kernel
 * (server/exllama_kernels/exllama_kernels/cuda_func/q4_matrix.cu:166-220); used by the
 * parity tests and by callers that want a dense copy.
 */
int q4_dequant(const q4_weight* w, void* w_out, int dtype, void* stream);

/*
 * y = x @ W (+ bias).  The forward of the quantized linear layer; picks the decode or
 * the prefill kernel from M.  Replaces `gemm_half_q_half` (server/exllamav2_kernels/
 * exllamav2_kernels/ext.cpp:100-131 -> cuda/q_gemm.cu:116-191), `q4_matmul`
 * (server/exllama_kernels/exllama_kernels/exllama_ext.cpp:168-213), the Triton
 * `matmul248` launcher (server/text_generation_server/layers/gptq/triton.py:204-241)
 * and `awq_inference_engine.gemm_forward_cuda` (call site
 * server/text_generation_server/layers/awq/quantize/cuda.py:45-47).
 *
 * workspace: device buffer of at least q4_workspace_bytes(M, K, N) bytes whose first
 * Q4_WORKSPACE_COUNTER_BYTES bytes (split-K tickets, then fixed-point accumulation cells)
 * were zero before the first call that used it; the kernels leave them zero again.  The
 * rest holds fp32 partial sums and needs no initialisation.  Calls that share a workspace
 * must be ordered on one stream.
 */
int q4_linear(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
              void* workspace, size_t workspace_bytes, void* stream);

/* Same as q4_linear with the kernel path forced (Q4_PATH_*); for tests and benchmarks. */
int q4_linear_ex(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                 void* workspace, size_t workspace_bytes, int path, void* stream);

/*
 * First half of a gated MLP in one launch: W packs [gate | up] along N and
 *   y[M, N/2] = act(x @ gate (+ bias[:N/2])) * (x @ up (+ bias[N/2:])),
 * with the roundings of the unfused sequence (both products rounded to `dtype`, the
 * activation evaluated in fp32 and rounded, the product rounded).  Replaces
 * `gate_up_proj(x)` followed by `act(gate_up[:, 0]) * gate_up[:, 1]`
 * (server/text_generation_server/models/custom_modeling/flash_llama_modeling.py:400-404;
 * the reference fuses this only for unquantized ROCm decode, `ops.LLMM_Silu`, :378-397).
 * Fused in the decode kernel of the GPTQ layout with contiguous groups.  Returns
 * Q4_ERR_UNSUPPORTED otherwise (AWQ layout, g_idx, odd shapes, and M large enough for the
 * prefill GEMM, where the separate elementwise pass is the faster route): the caller then
 * runs q4_linear into an [M, N] buffer and q4_act_mul.
 */
#define Q4_ACT_SILU 0       /* x * sigmoid(x) */
#define Q4_ACT_GELU_TANH 1  /* gelu(approximate="tanh"): "gelu_fast", "gelu_pytorch_tanh" */
#define Q4_ACT_GELU 2       /* gelu(approximate="none") */
int q4_linear_gate_up(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                      int act, void* workspace, size_t workspace_bytes, void* stream);

/*
 * Which route is faster for the gated first half of an MLP on this problem: *fused = 1 when a
 * fused kernel exists (q4_linear_gate_up will run) and it measured faster than q4_linear into an
 * [M, N] buffer followed by q4_act_mul, else 0.  A pure function of (w's geometry, M, dtype).
 */
int q4_linear_gate_up_plan(const q4_weight* w, int M, int dtype, int* fused);

/*
 * Act-order by row order instead of per-weight lookups, as the reference's exllamav2 path does
 * (QMatrix::make_sequential and make_sequential_kernel,
 * server/exllamav2_kernels/exllamav2_kernels/cuda/q_matrix.cu:524-640; activations read
 * through b_q_perm, cuda/q_gemm_kernel_gptq.cuh:116).  With perm = a stable argsort of g_idx,
 * q4_gptq_make_sequential writes qweight_out whose packed row i holds checkpoint row perm[i]
 * (GPTQ layout, [K/8, N], once at load time; qzeros and scales are unchanged).  When every group
 * has exactly `groupsize` rows the result is a contiguous-group matrix: pass it with g_idx = NULL
 * and feed q4_linear the activations in the same order, x_seq[m][i] = x[m][perm[i]], which
 * q4_gather_columns produces (16-bit elements, [M, K], K a multiple of 8).  Indices outside
 * 0..K-1 are clamped.
 */
int q4_gptq_make_sequential(const uint32_t* qweight, const int32_t* perm, uint32_t* qweight_out, int K, int N,
                            void* stream);
int q4_gather_columns(const void* x, const int32_t* perm, void* out, int M, int K, void* stream);
/*
 * q4_linear for a weight in group order, x in checkpoint order: y = x[:, perm] @ W (+ bias).
 * With a few rows and K <= 4096 the decode kernel reads x through perm while it stages it
 * (no extra pass, as the reference's kernel does with b_q_perm); otherwise x is gathered once
 * into the tail of the workspace, which therefore must hold q4_workspace_bytes_perm(M, K, N)
 * bytes (its head is the zero-initialised area of q4_workspace_bytes).  `path` as for q4_linear_ex; perm NULL
 * makes this q4_linear_ex.
 */
int q4_linear_perm(const q4_weight* w, const int32_t* perm, const void* x, const void* bias, void* y, int M,
                   int dtype, void* workspace, size_t workspace_bytes, int path, void* stream);
size_t q4_workspace_bytes_perm(int M, int K, int N);
/* q4_linear_gate_up for a weight in group order, x in checkpoint order (see q4_linear_perm);
 * Q4_ERR_UNSUPPORTED where the fused kernel does not apply: then q4_linear_perm + q4_act_mul. */
int q4_linear_gate_up_perm(const q4_weight* w, const int32_t* perm, const void* x, const void* bias, void* y, int M,
                           int dtype, int act, void* workspace, size_t workspace_bytes, void* stream);
/*
 * One block of the GPTQ solver's column loop (GPTQ.fasterquant,
 * server/text_generation_server/layers/gptq/quantize.py:294-331; the quantizer's range rule,
 * Quantizer.find_params, :60-101 with mse off, and its rounding, :54-58).  W [rows, K] fp32
 * holds the current weights (one row per output feature); U [K, K] is the upper Cholesky factor
 * of the inverse damped Hessian.  For the columns i1 .. i1+count-1 (count <= 128) in turn:
 * at a group start find scale and zero of the group from the current values, quantize the
 * column to 4 bits, store scale*(q - zero) in Q, (w - q) / U_ii in err [rows, 128], add
 * (w - q)^2 / U_ii^2 / 2 to loss [rows], and subtract err * U[i, c] from every later column c
 * of the block.  W itself is not written; the caller follows with
 * W[:, i1+count:] -= err @ U[i1:i1+count, i1+count:].  groupsize <= 0: scale / zero [rows]
 * are given; else they are [rows, num_groups] and the groups starting in the block are written.
 * sym: bit 0 = symmetric range; bit 1 = the parameters of the groups that start in the block
 * are given too (the caller found them, e.g. with the quantizer's mse search, :101-123, from
 * W as it is when the block starts) and the kernel only reads them.
 */
int q4_gptq_solve_block(float* W, const float* U, float* Q, float* err, float* loss, float* scale, float* zero,
                        int rows, int K, int i1, int count, int groupsize, int num_groups, int sym, void* stream);

/*
 * Grouped form of q4_gather_columns for experts whose rows are in group order (perms [E, K],
 * one q4_gptq_make_sequential per expert): out[r][i] = x[x_rows ? x_rows[r] : r][perms[e(r)][i]]
 * for every sorted row r, e(r) its expert by expert_offsets.  out is [pairs, K] in sorted order
 * and goes to q4_moe_linear with x_rows = NULL.
 */
int q4_moe_gather_columns(const void* x, const int32_t* x_rows, const int32_t* expert_offsets, const int32_t* perms,
                          void* out, int num_experts, int pairs, int K, void* stream);

/* y[M, inter] = act(gate_up[:, :inter]) * gate_up[:, inter:] for gate_up [M, 2 * inter]. */
int q4_act_mul(const void* gate_up, void* y, int M, int inter, int dtype, int act, void* stream);

/*
 * Decode kernel with an explicit work decomposition, for tuning sweeps and measured plans:
 * `wcol` waves across columns and `wk` waves across K per workgroup (wcol * wk <= 8), `splits`
 * workgroups across K, `words` packed words per lane (4, 2 or 1: column tiles of 64, 32 or
 * 16 per wave; GPTQ layout with contiguous groups of at least 128 rows, otherwise forced to
 * 4; the AWQ kernel's tile is 256 columns; 0: the instruction-lean kernel / the AWQ kernel that
 * feeds the stored words to the matrix core; -1: the short-launch kernel for up to 16 rows of
 * contiguous GPTQ groups, wcol unused).  N must be a multiple of tile * wcol.
 * Plays the role of exllama's `set_tuning_params`
 * (server/exllama_kernels/exllama_kernels/exllama_ext.cpp:78-100) without global state.
 */
int q4_gemv_tuned(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                  void* workspace, size_t workspace_bytes, int wcol, int wk, int splits, int words,
                  void* stream);

/*
 * Decode decompositions worth timing for this problem at load time, as (wcol, wk, splits, words)
 * quadruples for q4_gemv_tuned, written to configs[4 * i ..]; returns how many (0 when q4_linear
 * would not run a decode kernel here or no alternative to its own choice exists), at most
 * max_configs.  A caller that wants measured instead of fitted plans times q4_linear and each
 * candidate on its own weights once per layer shape and row count and keeps the winner (the
 * Python layers do so in their Warmup hook).  Plays the role of the autotuner of the reference's
 * Triton path (server/text_generation_server/layers/gptq/custom_autotune.py:1-80, the config
 * list of layers/gptq/triton.py:14-103).  GPTQ weights with contiguous groups: decompositions
 * of the short-launch kernel (words = -1); AWQ weights up to 8 rows: of the words-as-stored kernel
 * (words = 0).  A candidate whose activations do not fit LDS makes q4_gemv_tuned return
 * Q4_ERR_UNSUPPORTED; skip it.  q4_gemv_tuned_workspace_bytes: workspace such a call needs (the
 * zero-initialised head included).
 */
int q4_gemv_candidates(const q4_weight* w, int M, int dtype, int32_t* configs, int max_configs);
size_t q4_gemv_tuned_workspace_bytes(const q4_weight* w, int M, int dtype, int wcol, int wk, int splits, int words);

/*
 * Bytes of workspace q4_linear needs for an [M, K] x [K, N] problem (split-K partial
 * sums + ticket counters).  Replaces the scratch sizing of
 * server/text_generation_server/layers/gptq/exllamav2.py:233-240
 * (temp_dq_size / temp_fwd_size / scratch_space_fixed).
 */
#define Q4_WORKSPACE_TICKET_BYTES 16384   /* split-K arrival tickets, one per column tile */
#define Q4_WORKSPACE_CELL_BYTES 4194304   /* 64-bit fixed-point accumulation cells (fp16 decode: 16 rows x 32768 columns) */
#define Q4_WORKSPACE_COUNTER_BYTES 4210688 /* = tickets + cells: the part that must start zero */
size_t q4_workspace_bytes(int M, int K, int N);
/*
 * The same for one weight: exactly what q4_linear / q4_linear_gate_up need for `w` at M rows
 * (either dtype).  q4_workspace_bytes is an upper bound over every weight of the shape.
 */
size_t q4_workspace_bytes_for(const q4_weight* w, int M);
/*
 * Everything a caller needs to know before q4_linear_ex(w, ..., M, dtype, ...) in one call:
 * *path = q4_select_path(w, M, dtype), *workspace_bytes = q4_workspace_bytes_for(w, M).  Both are
 * pure functions of (w's geometry, M, dtype): a caller may keep them per layer and batch size
 * and pass `path` to q4_linear_ex.  Replaces the per-layer sizing the reference does once at
 * Warmup (server/text_generation_server/layers/gptq/exllamav2.py:159-175, 233-240).
 */
int q4_linear_plan(const q4_weight* w, int M, int dtype, int* path, size_t* workspace_bytes);

/*
 * q4_linear for callers that cannot allocate device memory or hand over a workspace (code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc).  No
 * counterpart in the reference.  The split-K scratch (tickets, accumulation cells, fp32
 * partial sums) lives in a device array built into the library, Q4_NOALLOC_SCRATCH_BYTES per
 * GPU, held until the process ends; the call allocates and frees nothing.  Decode problems
 * whose partial sums do not fit return Q4_ERR_WORKSPACE (q4_linear_plan tells the size);
 * prefill problems run unsplit where their partial tiles do not fit.  All calls on one GPU
 * share the array: calls that overlap on one GPU (two streams) race; the kernels leave the
 * counters at zero, so consecutive calls need no clearing.  q4_noalloc_init() looks the
 * array's address up for the current device (the first q4_linear_noalloc on a device does
 * it otherwise; call it before a stream capture begins).
 */
#define Q4_NOALLOC_SCRATCH_BYTES 16777216
int q4_noalloc_init(void);
int q4_linear_noalloc(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype, void* stream);

/*
 * ---- Mixture of experts: the same linear layer, grouped over experts -----------------
 *
 * Replaces, for GPTQ and AWQ checkpoints, what the reference's sparse MoE layer
 * (server/text_generation_server/layers/moe/gptq_marlin.py:116-146 -> fused_marlin_moe,
 * :232-351) gets from the un-vendored `kernels-community/moe` package (fused_topk +
 * fused_marlin_moe): routing, the two grouped projections and the weighted sum.  The
 * expert tensors stay in checkpoint layout (GPTQ with or without act-order, or AWQ), stacked along a leading expert dimension
 * (what _pack_weight, gptq_marlin.py:186-229, builds) -- there is no Marlin repack.
 *
 * Rows are (token, expert) pairs sorted by expert.  q4_moe_route writes, all on the
 * device and without a host round trip:
 *   topk_weights f32 [tokens, topk], topk_ids int32 [tokens, topk]   routing result
 *   sorted_tokens int32 [tokens*topk]   token of every sorted row
 *   pair_slot     int32 [tokens*topk]   sorted row of pair (t, j) = pair_slot[t*topk + j]
 *   expert_offsets int32 [experts + 1]  first sorted row of every expert
 * The order of the rows of one expert is not specified (no output depends on it).
 */
typedef struct q4_moe_weight {
  q4_weight expert0;      /* geometry and the tensors of expert 0 (either layout, g_idx optional) */
  int32_t num_experts;
  int64_t qweight_stride; /* elements between consecutive experts' qweight / qzeros / scales / g_idx */
  int64_t qzeros_stride;
  int64_t scales_stride;
  int64_t g_idx_stride;   /* ignored when expert0.g_idx is NULL */
} q4_moe_weight;

#define Q4_DTYPE_F32 2 /* gating logits only */

/* softmax over experts, top-k (ties: lowest expert), optional renormalisation to sum 1,
 * then the sort by expert described above.  experts <= 256, topk <= 8. */
int q4_moe_route(const void* gating, int gating_dtype, int tokens, int experts, int topk, int renormalize,
                 float* topk_weights, int32_t* topk_ids, int32_t* sorted_tokens, int32_t* pair_slot,
                 int32_t* expert_offsets, void* stream);

/* Grouped top-k (the in-tree definition: server/text_generation_server/layers/moe/
 * fused_moe_ipex.py:21-50): the experts form num_expert_group equal groups, a token keeps the
 * topk_group groups whose best expert scores highest and chooses its topk experts among those.
 * num_expert_group = 0: plain top-k.  At most 32 groups. */
int q4_moe_route_grouped(const void* gating, int gating_dtype, int tokens, int experts, int topk, int renormalize,
                         int num_expert_group, int topk_group, float* topk_weights, int32_t* topk_ids,
                         int32_t* sorted_tokens, int32_t* pair_slot, int32_t* expert_offsets, void* stream);

/* y[r, :] = x[x_rows ? x_rows[r] : r, :] @ W_e for every sorted row r of every expert e.
 * y is [tokens*topk, N] in sorted order.  Up to 16 tokens (64 when K <= 8192) the decode
 * kernel runs once per expert and 16 rows it received; above, the MFMA kernel.  Workspace as for q4_linear, sized by
 * q4_moe_workspace_bytes, zero-initialised once. */
int q4_moe_linear(const q4_moe_weight* w, const void* x, const int32_t* x_rows, const int32_t* expert_offsets,
                  void* y, int tokens, int topk, int dtype, void* workspace, size_t workspace_bytes, void* stream);

/* First projection with the gated-MLP epilogue: every expert's W packs [gate | up] along N and
 * y[r, :] = act(x_r @ gate_e) * (x_r @ up_e), [tokens*topk, N/2] in sorted order.  One launch
 * where the fused decode kernel applies (one token, GPTQ layout with contiguous groups
 * of at least 128 rows); Q4_ERR_UNSUPPORTED otherwise -- then q4_moe_linear + q4_act_mul. */
int q4_moe_linear_gate_up(const q4_moe_weight* w, const void* x, const int32_t* x_rows, const int32_t* expert_offsets,
                          void* y, int tokens, int topk, int dtype, int act, void* workspace, size_t workspace_bytes,
                          void* stream);

/* out[t, :] = sum_j topk_weights[t, j] * y_sorted[pair_slot[t*topk + j], :], summed in fp32
 * in the order j = 0, 1, ..., rounded once. */
int q4_moe_combine(const void* y_sorted, const float* topk_weights, const int32_t* pair_slot, void* out,
                   int tokens, int topk, int N, int dtype, void* stream);

size_t q4_moe_workspace_bytes(const q4_moe_weight* w, int tokens, int topk);

/* The Q4_PATH_* value q4_linear would take for this problem (negative on bad arguments). */
int q4_select_path(const q4_weight* w, int M, int dtype);

/* Message for the last failing call on this thread ("" if none). */
const char* q4_last_error(void);

/* ABI version; bumped when a signature changes. */
int q4_abi_version(void);

#ifdef __cplusplus
}
#endif
#endif /* Q4_LINEAR_H */
