// Shared device helpers for the int4 weight-only linear kernels (gfx950 / CDNA4 only).
//
// Nibble -> half conversion uses the exponent-splice identity: for 0 <= q <= 15 the
// fp16 bit pattern 0x6400 | q is exactly 1024 + q, and 0x6400 | (q << 4) is exactly
// 1024 + 16 q.  One 32-bit AND+OR therefore converts two nibbles that sit 16 bits apart
// (nibbles j and j+4 of a packed word) into a half2 with no integer->float conversion.
// The pairing (j, j+4) is kept all the way into the MFMA operand; the activation tile
// is permuted to the same order instead of repacking the weights.
#pragma once
#ifdef Q4_PHASE_STAMPS
// measurement build: waves per launch the phase-stamp buffer has room for
#define Q4_PHASE_STAMP_SLOTS 16384
#endif

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "q4_linear.h"

namespace q4 {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16_t;
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

// Logical column held at nibble position p of an AWQ word is 8c + kAwqOrder[p]
// (server/text_generation_server/layers/awq/conversion_utils.py:5).
__device__ __forceinline__ int awq_order(int p) { return ((p & 3) << 1) | (p >> 2); }
// Nibble position that holds logical column 8c + i (conversion_utils.py:6).
__device__ __forceinline__ int awq_position(int i) { return ((i & 1) << 2) | (i >> 1); }

__device__ __forceinline__ uint32_t as_u32(half2_t h) { return __builtin_bit_cast(uint32_t, h); }
__device__ __forceinline__ half2_t as_half2(uint32_t u) { return __builtin_bit_cast(half2_t, u); }

// (stored + 1) & 15 on eight packed nibbles at once (GPTQ zero-point rule,
// server/text_generation_server/layers/gptq/triton.py:184-185).
__device__ __forceinline__ uint32_t gptq_zero_plus_one(uint32_t z) {
  return ((z & 0x77777777u) + 0x11111111u) ^ (z & 0x88888888u);
}

// float -> bf16 bits, round to nearest even (inputs here are finite).
__device__ __forceinline__ uint16_t f32_to_bf16_rne(float f) {
  uint32_t u = __builtin_bit_cast(uint32_t, f);
  u += 0x7FFFu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  return __builtin_bit_cast(float, (uint32_t)b << 16);
}

// One dequantized weight in the reference's arithmetic: round_once(s * (q - z)).
// (q - z) is an exact small integer; in fp16 the single multiply rounds once
// (triton.py:192, q_matrix.cu:282-293); in bf16 the exact fp32 product is rounded once.
template <int DTYPE>
__device__ __forceinline__ uint16_t dequant_one(half_t s, int q, int z) {
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    half_t w = (half_t)(float)(q - z) * s;
    return __builtin_bit_cast(uint16_t, w);
  } else {
    return f32_to_bf16_rne((float)s * (float)(q - z));
  }
}

template <int DTYPE>
__device__ __forceinline__ float load_act(const void* p, size_t idx) {
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    return (float)((const half_t*)p)[idx];
  } else {
    return bf16_bits_to_f32(((const uint16_t*)p)[idx]);
  }
}

template <int DTYPE>
__device__ __forceinline__ uint16_t store_act(float v) {
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    half_t h = (half_t)v;
    return __builtin_bit_cast(uint16_t, h);
  } else {
    return f32_to_bf16_rne(v);
  }
}

// Output rounding used by every kernel: the fp32 sum is cast to the activation dtype,
// then the bias is added in that dtype's arithmetic (fp32 add, rounded once), matching
// `out + self.bias` on a half tensor (triton.py:362).
template <int DTYPE>
__device__ __forceinline__ uint16_t finish_output(float acc, const void* bias, int n) {
  uint16_t y = store_act<DTYPE>(acc);
  if (bias != nullptr) {
    float yb;
    if constexpr (DTYPE == Q4_DTYPE_F16) {
      yb = (float)__builtin_bit_cast(half_t, y) + (float)((const half_t*)bias)[n];
    } else {
      yb = bf16_bits_to_f32(y) + bf16_bits_to_f32(((const uint16_t*)bias)[n]);
    }
    y = store_act<DTYPE>(yb);
  }
  return y;
}

// Gated-MLP epilogue: act(gate) * up on values already rounded to the activation dtype, with
// the roundings of the unfused sequence `act(g) * u` on half tensors (the activation is
// evaluated in fp32 and rounded, then the product is rounded):
// server/text_generation_server/models/custom_modeling/flash_llama_modeling.py:400-404.
// `act` is a Q4_ACT_* value.
// ACT is a Q4_ACT_* value.  silu and the tanh form of gelu are both g * sigmoid(t) (t = g, or
// t = 2 * sqrt(2/pi) * (g + 0.044715 g^3): 0.5 * (1 + tanh(t/2)) is sigmoid(t), without the
// cancellation of 1 + tanh for negative inputs); the exponential and the reciprocal are the
// hardware ones (about 1 ulp each in fp32, far inside the half rounding that follows).
template <int ACT>
__device__ __forceinline__ float act_value(float g) {
  if constexpr (ACT == Q4_ACT_GELU) {
    return 0.5f * g * (1.0f + erff(g * 0.7071067811865476f));
  } else {
    // (written so that no multiply-add pair is left to the compiler's choice of contraction:
    // every kernel that inlines this rounds alike)
    float t = g;
    if constexpr (ACT == Q4_ACT_GELU_TANH) t = (1.5957691216057308f * g) * __builtin_fmaf(0.044715f, g * g, 1.0f);
    return g * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * t));
  }
}

template <int DTYPE, int ACT>
__device__ __forceinline__ uint16_t act_mul_as(uint16_t g_bits, uint16_t u_bits) {
  float g, u;
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    g = (float)__builtin_bit_cast(half_t, g_bits);
    u = (float)__builtin_bit_cast(half_t, u_bits);
  } else {
    g = bf16_bits_to_f32(g_bits);
    u = bf16_bits_to_f32(u_bits);
  }
  // The activation is rounded to fp32 and then to the half type, as an fp32 routine followed
  // by a cast does.  The empty asm keeps the compiler from folding the last multiply and the
  // cast into one mixed-precision multiply-add, which rounds once (and loses the sign of a
  // zero): every kernel that inlines this then gives the same bits.
  float a = act_value<ACT>(g);
  asm("" : "+v"(a));
  const uint16_t a_bits = store_act<DTYPE>(a);
  float ar;
  if constexpr (DTYPE == Q4_DTYPE_F16) ar = (float)__builtin_bit_cast(half_t, a_bits);
  else ar = bf16_bits_to_f32(a_bits);
  return store_act<DTYPE>(ar * u);
}

template <int DTYPE>
__device__ __forceinline__ uint16_t act_mul(uint16_t g_bits, uint16_t u_bits, int act) {
  if (act == Q4_ACT_SILU) return act_mul_as<DTYPE, Q4_ACT_SILU>(g_bits, u_bits);
  if (act == Q4_ACT_GELU_TANH) return act_mul_as<DTYPE, Q4_ACT_GELU_TANH>(g_bits, u_bits);
  return act_mul_as<DTYPE, Q4_ACT_GELU>(g_bits, u_bits);
}

// Kernel-side view of q4_weight plus the activation-side pointers.
struct Problem {
  const uint32_t* __restrict__ qweight;
  const uint32_t* __restrict__ qzeros;
  const half_t* __restrict__ scales;
  const int32_t* __restrict__ g_idx;
  const void* __restrict__ x;
  const void* __restrict__ bias;
  void* __restrict__ y;
  int M, K, N, groupsize, num_groups;
  // 0: y[M, N] = x @ W (+ bias).  Q4_ACT_* + 1: gated-MLP epilogue, W = [gate | up] along N
  // and y[M, N/2] = act(x @ gate (+ bias)) * (x @ up (+ bias)); only kernels that say so
  // support it.
  int gate_up_act;
  // Decode kernels only: column of x behind every K row (x_seq[m][k] = x[m][x_perm[k]], the
  // row order of a weight whose act-order rows were put into group order), or nullptr.
  const int32_t* __restrict__ x_perm;
};

// Grouped launch over the experts of a mixture-of-experts layer.  The rows of the problem are
// the (token, expert) pairs sorted by expert: expert e owns sorted rows offsets[e] ..
// offsets[e + 1] - 1, its tensors sit e * stride elements behind expert 0's, and it writes
// the same rows of y.  x_rows, when given, names the row of x every sorted row reads (the
// first projection reads tokens); otherwise x is in sorted order like y.
struct MoeView {
  const int32_t* __restrict__ offsets;  // [experts + 1], device memory
  const int32_t* __restrict__ x_rows;   // [pairs] or nullptr
  long qweight_stride, qzeros_stride, scales_stride, g_idx_stride;
};

// Narrows `p` to expert e.  Returns the expert's first sorted row; p.M becomes its row count
// (possibly 0).  With x_rows the activation pointer stays whole (rows are looked up).
__device__ __forceinline__ int moe_enter(Problem& p, const MoeView& mv, int e) {
  const int row0 = mv.offsets[e];
  p.M = mv.offsets[e + 1] - row0;
  p.qweight += (size_t)e * mv.qweight_stride;
  p.qzeros += (size_t)e * mv.qzeros_stride;
  p.scales += (size_t)e * mv.scales_stride;
  if (p.g_idx != nullptr) p.g_idx += (size_t)e * mv.g_idx_stride;
  p.y = (uint16_t*)p.y + (size_t)row0 * p.N;
  if (mv.x_rows == nullptr) p.x = (const uint16_t*)p.x + (size_t)row0 * p.K;
  return row0;
}

}  // namespace q4

// Host-side launchers implemented by the kernel translation units.
namespace q4host {
void set_error(const char* fmt, ...);
int launch_dequant(const q4_weight* w, void* w_out, int dtype, hipStream_t stream);
int launch_generic(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                   hipStream_t stream);
struct GemvConfig {
  int wcol;    // waves across columns in a workgroup (one column tile each)
  int wk;      // waves across K in a workgroup
  int splits;  // workgroups across K (cross-workgroup reduction through the workspace)
  int words;   // GPTQ contiguous-group kernel: packed words per lane (4, 2, 1 -> 64/32/16-column tiles)
  int rows_per_block = 16;  // 32: GPTQ contiguous-group kernel with two MFMA row blocks (17..32 rows)
  int lean = 0;  // 1: the instruction-lean contiguous-group kernel (groups of whole 128-row chunks, up to 16 waves)
};
bool gemv_lean_supported(const q4_weight* w, int dtype);
bool gemv_supported(const q4_weight* w, int M, int dtype);
bool gemv_rows32_supported(const q4_weight* w, int M);
bool gemv_rows32_kernel(const q4_weight* w, int M);
GemvConfig gemv_pick_config(const q4_weight* w, int M);
GemvConfig gemv_pick_config(const q4_weight* w, int M, bool gate_up);
int launch_gemv(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                void* workspace, size_t workspace_bytes, const GemvConfig* cfg, hipStream_t stream,
                int gate_up_act = 0, const int32_t* x_perm = nullptr);
// the short-launch decode kernel (q4_gemv_direct.cuh): up to 16 rows, contiguous GPTQ groups
bool gemv_direct_supported(const q4_weight* w, int M, int dtype, int wk, int splits);
size_t gemv_direct_workspace_bytes(const q4_weight* w, int M, int dtype, int splits);
bool gemv_direct_default(const q4_weight* w, int M, int dtype, int* wk, int* splits);
int launch_gemv_direct(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype, void* workspace,
                       size_t workspace_bytes, int wk, int splits, hipStream_t stream);
bool gemv_gate_up_supported(const q4_weight* w, int M, int dtype);
int launch_act_mul(const void* gate_up, void* y, int M, int inter, int dtype, int act, hipStream_t stream);
bool gemm_gate_up_supported(const q4_weight* w, int M, int dtype);
int launch_gemm_gate_up(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype, int act,
                        hipStream_t stream);
int launch_make_sequential(const uint32_t* qweight, const int32_t* perm, uint32_t* out, int K, int N, hipStream_t stream);
int launch_gather_columns(const void* x, const int32_t* perm, void* out, int M, int K, hipStream_t stream);
int launch_gptq_solve_block(float* W, const float* U, float* Q, float* Err, float* loss, float* scale, float* zero,
                            int rows, int K, int i1, int count, int groupsize, int G, int sym, hipStream_t stream);
int launch_moe_gather_columns(const void* x, const int32_t* x_rows, const int32_t* offsets, const int32_t* perms,
                              void* out, int num_experts, int pairs, int K, hipStream_t stream);
bool gemm_awq_supported(const q4_weight* w, int M, int dtype);
// Host description of a grouped (mixture-of-experts) launch.
struct MoeLaunch {
  q4::MoeView view;
  int num_experts;
  int tokens;  // an expert can receive at most this many rows
  int pairs;   // tokens * topk: rows of the sorted order
};
// moe != nullptr: grouped launch, M = moe->tokens, y and the partial tiles have moe->pairs rows
int launch_gemm_awq(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                    void* workspace, size_t workspace_bytes, hipStream_t stream, const MoeLaunch* moe = nullptr);
size_t gemm_awq_moe_workspace_bytes(const q4_weight* w, const MoeLaunch* moe);
// AWQ layout, dense launches: the kernel that unpacks the checkpoint words in registers
bool gemm_awq_direct_supported(const q4_weight* w, int M, int dtype);
int launch_gemm_awq_direct(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                           void* workspace, size_t workspace_bytes, hipStream_t stream);
size_t gemm_awq_direct_workspace_bytes(int M, int K, int N);
bool gemm_supported(const q4_weight* w, int M, int dtype);
int launch_gemm(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                void* workspace, size_t workspace_bytes, hipStream_t stream);
size_t gemm_workspace_bytes(int M, int K, int N);
// Split factor of an under-filled tile grid from the fitted cost model (us per K tile of a
// workgroup alone on its CU / sharing it).
int gemm_pick_splits(long tiles, int KT, int M, int N, double us_alone, double us_shared, int per_cu = 2);
bool gemm_act_order_table(const q4_weight* w);  // act-order GEMM reads its parameters from LDS
int gemm_awq_splits(int M, int K, int N, bool one_per_cu, bool tall = false);
void launch_gemm_reduce(const float* partials, const void* bias, void* y, int M, int N, int splits, int dtype,
                        hipStream_t stream);
}  // namespace q4host
