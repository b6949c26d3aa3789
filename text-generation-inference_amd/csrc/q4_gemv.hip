// Decode path: y[M<=16, N] = x @ dequant(W), GPTQ layout, groups contiguous in K.
//
// HBM-bound: the packed weights are read exactly once with 128-bit loads and never
// written back.  Work decomposition (all wave64):
//   * a wave owns 64 columns; lane l covers columns n0 + 4*(l%16) .. +3 and the packed row
//     r0 + l/16, so one global_load_dwordx4 per lane fetches a 4-row x 256-byte patch
//     (32 K rows x 64 columns) whose rows are contiguous 256-byte segments;
//   * a packed word already holds 8 consecutive K values of one column, which is exactly
//     what one lane of a 16x16x32 MFMA supplies for the B operand (column l%16, K block
//     l/16).  Word t of the dwordx4 feeds MFMA t; the four MFMAs produce columns
//     n0 + 4*j + t.  The matrix core performs both the multiply and the reduction across
//     the four K blocks of the wave, so the VALU only unpacks nibbles;
//   * nibbles become halves with one AND+OR each pair (see q4_common.cuh) in the order
//     [0,4,1,5,2,6,3,7]; the activation slab is staged once per workgroup in LDS in that
//     same order, so no weight is ever repacked;
//   * zero points are subtracted exactly in fp16 ((1024+q) - (1024+z)); the group scale
//     is factored out of the K sum and applied to the fp32 group accumulator, so a weight
//     costs ~1.1 VALU operations;
//   * split-K: `wk` waves of a workgroup take consecutive K ranges and are combined
//     through LDS in fixed order; `splits` workgroups write fp32 partials to the
//     workspace and the last one to arrive (ticket counter) adds them in split order and
//     writes the output.  The result is deterministic and needs no memset: the last
//     workgroup resets its ticket.
// Workgroup ids are laid out split-major so that all splits of a column tile land on the
// same XCD (id % 8) and the partials stay in that XCD's L2.
#include "q4_common.cuh"

namespace q4 {

constexpr int kChunkSteps = 4;              // 32-row MFMA steps per software-pipelined chunk
constexpr int kChunkRows = 32 * kChunkSteps;  // 128 K rows

struct GemvParams {
  Problem p;
  float* __restrict__ partials;
  uint32_t* __restrict__ tickets;
  int wcol, wk, splits;
  int slab_stride;  // bytes between activation rows in LDS
};

__device__ __forceinline__ uint32_t nib_lo(uint32_t w) { return (w & 0x000F000Fu) | 0x64006400u; }
__device__ __forceinline__ uint32_t nib_hi(uint32_t w) { return (w & 0x00F000F0u) | 0x64006400u; }

// Eight exact (q - z) values of one packed word, as four half2 in K order [0,4,1,5,2,6,3,7].
// czlo = half2(-(1024 + z)), czhi = half2(-(64 + z)).
__device__ __forceinline__ void unpack_word_f16(uint32_t w, half2_t czlo, half2_t czhi,
                                                half2_t out[4]) {
  const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  const uint32_t w8 = w >> 8;
  out[0] = as_half2(nib_lo(w)) + czlo;
  out[1] = as_half2(nib_hi(w)) * sixteenth + czhi;
  out[2] = as_half2(nib_lo(w8)) + czlo;
  out[3] = as_half2(nib_hi(w8)) * sixteenth + czhi;
}

__device__ __forceinline__ uint32_t pack_bf16_pair(half2_t h) {
  // Small integers are exact in fp32 with a zero low half, so truncation is exact.
  const uint32_t lo = __builtin_bit_cast(uint32_t, (float)h.x);
  const uint32_t hi = __builtin_bit_cast(uint32_t, (float)h.y);
  return (lo >> 16) | (hi & 0xFFFF0000u);
}

template <int DTYPE>
__device__ __forceinline__ float4_t mfma16(const uint4_t a, const half2_t b[4], float4_t c) {
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    union {
      half2_t h[4];
      half8_t v;
    } bu;
    bu.h[0] = b[0]; bu.h[1] = b[1]; bu.h[2] = b[2]; bu.h[3] = b[3];
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), bu.v, c, 0, 0, 0);
  } else {
    uint4_t bb;
    bb.x = pack_bf16_pair(b[0]);
    bb.y = pack_bf16_pair(b[1]);
    bb.z = pack_bf16_pair(b[2]);
    bb.w = pack_bf16_pair(b[3]);
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, bb), c, 0, 0, 0);
  }
}

// GSTEPS: MFMA steps (32 rows) per quantisation group inside a chunk: 1, 2 or 4.
// STATIC128: groupsize is exactly 128, so every chunk is one whole group.
template <int DTYPE, int RMAX, int GSTEPS, bool STATIC128>
__global__ __launch_bounds__(512) void gemv_gptq_kernel(GemvParams gp) {
  extern __shared__ __align__(16) unsigned char smem[];
  const Problem& p = gp.p;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wc = wave % gp.wcol;
  const int wkk = wave / gp.wcol;
  const int j = lane & 15;
  const int kq = lane >> 4;
  const int nthreads = blockDim.x;

  const int tile_cols = 64 * gp.wcol;
  const int ntiles = p.N / tile_cols;
  const int tile = blockIdx.x % ntiles;
  const int split = blockIdx.x / ntiles;
  const int nl = tile * tile_cols + wc * 64 + 4 * j;  // first of this lane's 4 columns

  const int KR = p.K / gp.splits;  // rows of this workgroup
  const int KW = KR / gp.wk;       // rows of this wave
  const int kwg0 = split * KR;
  const int kw0 = kwg0 + wkk * KW;
  const int nchunks = KW / kChunkRows;
  const int N = p.N;
  constexpr int GPC = kChunkSteps / GSTEPS;  // groups per chunk

  // ---- issue the first chunk of weight loads before anything else
  const uint4_t* qw = (const uint4_t*)(p.qweight + (size_t)(kw0 / 8 + kq) * N + nl);
  const size_t step_stride = (size_t)N;  // uint4 units between consecutive 32-row steps
  uint4_t wq[kChunkSteps], wq_next[kChunkSteps];
#pragma unroll
  for (int s = 0; s < kChunkSteps; ++s) wq[s] = __builtin_nontemporal_load(qw + s * step_stride);

  const int zshift = (nl & 4) * 4;
  auto load_group = [&](int k, uint2_t& sc, uint32_t& zw) {
    int g = k / p.groupsize;
    g = min(g, p.num_groups - 1);
    sc = *(const uint2_t*)(p.scales + (size_t)g * N + nl);
    zw = p.qzeros[(size_t)g * (N >> 3) + (nl >> 3)];
  };
  uint2_t sc[GPC], sc_next[GPC];
  uint32_t zw[GPC], zw_next[GPC];
#pragma unroll
  for (int g = 0; g < GPC; ++g) load_group(kw0 + g * GSTEPS * 32, sc[g], zw[g]);

  // ---- stage the activation slab [M][KR] into LDS, each 8-block in order 0,4,1,5,2,6,3,7
  {
    const int kb_per_row = KR >> 3;
    const int total = p.M * kb_per_row;
    const uint16_t* xs = (const uint16_t*)p.x;
    for (int idx = tid; idx < total; idx += nthreads) {
      const int m = idx / kb_per_row;
      const int kb = idx - m * kb_per_row;
      const uint4_t v = *(const uint4_t*)(xs + (size_t)m * p.K + kwg0 + kb * 8);
      uint4_t o;
      o.x = (v.x & 0xFFFFu) | (v.z << 16);
      o.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
      o.z = (v.y & 0xFFFFu) | (v.w << 16);
      o.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
      *(uint4_t*)(smem + (size_t)m * gp.slab_stride + kb * 16) = o;
    }
  }
  __syncthreads();

  const bool row_live = j < p.M;  // A-operand row of this lane
  const unsigned char* a_base = smem + (size_t)j * gp.slab_stride + (size_t)(wkk * KW + kq * 8) * 2;

  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  float4_t tot[4] = {zero4, zero4, zero4, zero4};
  float4_t acc[4] = {zero4, zero4, zero4, zero4};
  half2_t czlo[4], czhi[4];

  for (int c = 0; c < nchunks; ++c) {
    const int kc = kw0 + c * kChunkRows;
    if (c + 1 < nchunks) {
#pragma unroll
      for (int s = 0; s < kChunkSteps; ++s)
        wq_next[s] = __builtin_nontemporal_load(qw + (size_t)((c + 1) * kChunkSteps + s) * step_stride);
#pragma unroll
      for (int g = 0; g < GPC; ++g) load_group(kc + kChunkRows + g * GSTEPS * 32, sc_next[g], zw_next[g]);
    }
    bool group_start, group_end;
    if constexpr (STATIC128) {
      group_start = true;
      group_end = true;
    } else if constexpr (GSTEPS == kChunkSteps) {
      group_start = (c == 0) || (kc % p.groupsize == 0);
      group_end = (c == nchunks - 1) || ((kc + kChunkRows) % p.groupsize == 0);
    } else {
      group_start = true;
      group_end = true;
    }
#pragma unroll
    for (int s = 0; s < kChunkSteps; ++s) {
      const int gi = s / GSTEPS;
      const bool first = (s % GSTEPS) == 0;
      const bool last = (s % GSTEPS) == GSTEPS - 1;
      if (first && (GSTEPS != kChunkSteps || group_start || STATIC128)) {
        // zero-point constants of the group: z = (stored + 1) & 15 per column
        const uint32_t z4 = gptq_zero_plus_one(zw[gi]) >> zshift;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t z = (z4 >> (4 * t)) & 0xFu;
          czlo[t] = as_half2(0xE400E400u | z | (z << 16));        // -(1024 + z)
          czhi[t] = as_half2(0xD400D400u | (z << 4) | (z << 20));  // -(64 + z)
        }
      }
      uint4_t a = {0u, 0u, 0u, 0u};
      if (row_live) a = *(const uint4_t*)(a_base + (size_t)(c * kChunkRows + s * 32) * 2);
      const uint32_t words[4] = {wq[s].x, wq[s].y, wq[s].z, wq[s].w};
      const bool fresh = first && (STATIC128 || GSTEPS != kChunkSteps);
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        half2_t b[4];
        unpack_word_f16(words[t], czlo[t], czhi[t], b);
        if (fresh) {
          acc[t] = mfma16<DTYPE>(a, b, zero4);
        } else {
          if (first && group_start) acc[t] = zero4;
          acc[t] = mfma16<DTYPE>(a, b, acc[t]);
        }
      }
      if (last && (GSTEPS != kChunkSteps || group_end || STATIC128)) {
        const half2_t s01 = as_half2(sc[gi].x), s23 = as_half2(sc[gi].y);
        const float sf[4] = {(float)s01.x, (float)s01.y, (float)s23.x, (float)s23.y};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
          for (int r = 0; r < RMAX; ++r) tot[t][r] = fmaf(sf[t], acc[t][r], tot[t][r]);
        }
      }
    }
#pragma unroll
    for (int s = 0; s < kChunkSteps; ++s) wq[s] = wq_next[s];
#pragma unroll
    for (int g = 0; g < GPC; ++g) {
      sc[g] = sc_next[g];
      zw[g] = zw_next[g];
    }
  }

  // ---- combine the wk waves of the workgroup through LDS (fixed order)
  if (gp.wk > 1) {
    __syncthreads();  // everyone is done with the activation slab
    float* red = (float*)smem;
    if (wkk > 0) {
      float* dst = red + ((size_t)((wkk - 1) * gp.wcol + wc) * 4 * RMAX) * 64 + lane;
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int r = 0; r < RMAX; ++r) dst[(t * RMAX + r) * 64] = tot[t][r];
    }
    __syncthreads();
    if (wkk == 0) {
      for (int w = 1; w < gp.wk; ++w) {
        const float* src = red + ((size_t)((w - 1) * gp.wcol + wc) * 4 * RMAX) * 64 + lane;
#pragma unroll
        for (int t = 0; t < 4; ++t)
#pragma unroll
          for (int r = 0; r < RMAX; ++r) tot[t][r] += src[(t * RMAX + r) * 64];
      }
    }
  }

  uint16_t* y = (uint16_t*)p.y;
  if (gp.splits == 1) {
    if (wkk == 0) {
#pragma unroll
      for (int r = 0; r < RMAX; ++r) {
        const int m = 4 * kq + r;
        if (m < p.M) {
          uint16_t o[4];
#pragma unroll
          for (int t = 0; t < 4; ++t) o[t] = finish_output<DTYPE>(tot[t][r], p.bias, nl + t);
          uint2_t packed;
          packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
          *(uint2_t*)(y + (size_t)m * N + nl) = packed;
        }
      }
    }
    return;
  }

  // ---- cross-workgroup split-K: write the partial, take a ticket, last one reduces
  if (wkk == 0) {
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      const int m = 4 * kq + r;
      if (m < p.M) {
        float4_t v = {tot[0][r], tot[1][r], tot[2][r], tot[3][r]};
        *(float4_t*)(gp.partials + ((size_t)split * p.M + m) * N + nl) = v;
      }
    }
  }
  __threadfence();
  __syncthreads();
  __shared__ uint32_t ticket_s;
  if (tid == 0) {
    ticket_s = __hip_atomic_fetch_add(gp.tickets + tile, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (ticket_s != (uint32_t)(gp.splits - 1)) return;
  __threadfence();
  {
    const int quads = tile_cols >> 2;
    const int items = p.M * quads;
    const int nbase = tile * tile_cols;
    for (int idx = tid; idx < items; idx += nthreads) {
      const int m = idx / quads;
      const int n = nbase + (idx - m * quads) * 4;
      float4_t sum = zero4;
      for (int s = 0; s < gp.splits; ++s) {
        const float4_t v = *(const float4_t*)(gp.partials + ((size_t)s * p.M + m) * N + n);
        sum += v;
      }
      uint16_t o[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) o[t] = finish_output<DTYPE>(sum[t], p.bias, n + t);
      uint2_t packed;
      packed.x = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
      packed.y = (uint32_t)o[2] | ((uint32_t)o[3] << 16);
      *(uint2_t*)(y + (size_t)m * N + n) = packed;
    }
    if (tid == 0) __hip_atomic_store(gp.tickets + tile, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

}  // namespace q4

namespace q4host {

using q4::GemvParams;
using q4::Problem;

bool gemv_supported(const q4_weight* w, int M, int dtype) {
  (void)dtype;
  if (w->layout != Q4_LAYOUT_GPTQ || w->g_idx != nullptr) return false;
  if (M < 1 || M > 16) return false;
  if (w->K % 128 != 0 || w->N % 64 != 0) return false;
  const int gs = w->groupsize;
  if (!(gs == 32 || gs == 64 || (gs >= 128 && gs % 128 == 0))) return false;
  if ((long)w->num_groups * gs < w->K) return false;
  if (w->N / 64 > Q4_WORKSPACE_COUNTER_BYTES / 4) return false;
  return true;
}

GemvConfig gemv_pick_config(const q4_weight* w, int M) {
  // Enough workgroups to cover 256 CUs several times over, each wave streaming at least
  // one 128-row chunk, with the activation slab (M rows x K/splits) inside 60 KB of LDS.
  GemvConfig c;
  const int chunks = w->K / 128;
  c.wcol = (w->N % 256 == 0) ? 4 : (w->N % 128 == 0 ? 2 : 1);
  c.wk = 1;
  const int ntiles = w->N / (64 * c.wcol);
  const int target_wgs = M <= 4 ? 1024 : 512;  // partial-sum traffic grows with M
  int want = (target_wgs + ntiles - 1) / ntiles;
  if (want > 32) want = 32;
  if (want < 1) want = 1;
  const long lds_budget = 60000 - 16L * M;
  int min_splits = (int)(((long)M * w->K * 2 + lds_budget - 1) / lds_budget);
  if (min_splits < 1) min_splits = 1;
  int best = chunks;  // always legal: one chunk per workgroup
  long best_cost = -1;
  for (int d = 1; d <= chunks; ++d) {
    if (chunks % d != 0 || d < min_splits) continue;
    const long cost = d > want ? (long)d * 1000 / want : (long)want * 1000 / d;
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = d;
    }
  }
  c.splits = best;
  return c;
}

template <int DTYPE, int RMAX>
static void launch_rmax(const GemvParams& gp, int gs, dim3 grid, dim3 block, size_t smem,
                        hipStream_t stream) {
  using namespace q4;
  if (gs == 128) {
    hipLaunchKernelGGL((gemv_gptq_kernel<DTYPE, RMAX, 4, true>), grid, block, smem, stream, gp);
  } else if (gs > 128) {
    hipLaunchKernelGGL((gemv_gptq_kernel<DTYPE, RMAX, 4, false>), grid, block, smem, stream, gp);
  } else if (gs == 64) {
    hipLaunchKernelGGL((gemv_gptq_kernel<DTYPE, RMAX, 2, false>), grid, block, smem, stream, gp);
  } else {
    hipLaunchKernelGGL((gemv_gptq_kernel<DTYPE, RMAX, 1, false>), grid, block, smem, stream, gp);
  }
}

int launch_gemv(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                void* workspace, size_t workspace_bytes, const GemvConfig* cfg_in,
                hipStream_t stream) {
  using namespace q4;
  if (!gemv_supported(w, M, dtype)) {
    set_error("q4_linear(gemv): unsupported problem (layout=%d g_idx=%p M=%d K=%d N=%d groupsize=%d)",
              w->layout, (const void*)w->g_idx, M, w->K, w->N, w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  const GemvConfig cfg = cfg_in ? *cfg_in : gemv_pick_config(w, M);
  if (cfg.wcol < 1 || cfg.wk < 1 || cfg.splits < 1 || cfg.wcol * cfg.wk > 8 ||
      w->N % (64 * cfg.wcol) != 0 || w->K % (cfg.splits * cfg.wk * 128) != 0) {
    set_error("q4_linear(gemv): bad config wcol=%d wk=%d splits=%d for K=%d N=%d", cfg.wcol, cfg.wk,
              cfg.splits, w->K, w->N);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  const int KR = w->K / cfg.splits;
  const int slab_stride = KR * 2 + 16;
  const int rmax = M <= 1 ? 1 : (M <= 2 ? 2 : 4);
  size_t smem = (size_t)M * slab_stride;
  const size_t red = (size_t)(cfg.wk - 1) * cfg.wcol * 4 * rmax * 64 * sizeof(float);
  if (red > smem) smem = red;
  if (smem > 64 * 1024) {
    set_error("q4_linear(gemv): config needs %zu bytes of LDS (> 64 KB)", smem);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  const int ntiles = w->N / (64 * cfg.wcol);
  float* partials = nullptr;
  uint32_t* tickets = nullptr;
  if (cfg.splits > 1) {
    const size_t need = Q4_WORKSPACE_COUNTER_BYTES + (size_t)cfg.splits * M * w->N * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need) {
      set_error("q4_linear(gemv): workspace of %zu bytes needed, %zu given", need, workspace_bytes);
      return Q4_ERR_WORKSPACE;
    }
    tickets = (uint32_t*)workspace;
    partials = (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES);
  }
  GemvParams gp;
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, nullptr, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  gp.partials = partials;
  gp.tickets = tickets;
  gp.wcol = cfg.wcol;
  gp.wk = cfg.wk;
  gp.splits = cfg.splits;
  gp.slab_stride = slab_stride;
  dim3 grid((unsigned)(ntiles * cfg.splits));
  dim3 block((unsigned)(64 * cfg.wcol * cfg.wk));
  const int gs = w->groupsize;
  if (dtype == Q4_DTYPE_F16) {
    if (rmax == 1) launch_rmax<Q4_DTYPE_F16, 1>(gp, gs, grid, block, smem, stream);
    else if (rmax == 2) launch_rmax<Q4_DTYPE_F16, 2>(gp, gs, grid, block, smem, stream);
    else launch_rmax<Q4_DTYPE_F16, 4>(gp, gs, grid, block, smem, stream);
  } else {
    if (rmax == 1) launch_rmax<Q4_DTYPE_BF16, 1>(gp, gs, grid, block, smem, stream);
    else if (rmax == 2) launch_rmax<Q4_DTYPE_BF16, 2>(gp, gs, grid, block, smem, stream);
    else launch_rmax<Q4_DTYPE_BF16, 4>(gp, gs, grid, block, smem, stream);
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemv): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
