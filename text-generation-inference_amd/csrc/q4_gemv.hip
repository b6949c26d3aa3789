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
constexpr int kPrefetch = 4;                  // chunks of weight loads in flight per wave

struct GemvParams {
  Problem p;
  float* __restrict__ partials;
  uint32_t* __restrict__ tickets;
  int wcol, wk, splits;
  int slab_stride;  // bytes between activation rows in LDS
};

// Constants of the nibble splice, hidden from constant folding (empty asm, no instruction
// is emitted): as literals the compiler must split (w & mask) | magic into v_and + v_or
// because a three-operand VALU instruction cannot carry a literal; as register operands it
// selects the fused v_and_or_b32.  The asm must stay empty: an instruction inside inline
// asm is invisible to the MFMA hazard recognizer.
struct SpliceConsts {
  uint32_t mask_lo, mask_hi, magic;
};
__device__ __forceinline__ SpliceConsts splice_consts() {
  SpliceConsts k{0x000F000Fu, 0x00F000F0u, 0x64006400u};
  asm volatile("" : "+s"(k.mask_lo), "+s"(k.mask_hi), "+v"(k.magic));
  return k;
}

// Eight exact (q - z) values of one packed word, as four half2 in K order [0,4,1,5,2,6,3,7].
// czlo = half2(-(1024 + z)), czhi = half2(-(64 + z)).
__device__ __forceinline__ void unpack_word_f16(uint32_t w, half2_t czlo, half2_t czhi,
                                                const SpliceConsts& k, half2_t out[4]) {
  const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  const uint32_t w8 = w >> 8;
  out[0] = as_half2((w & k.mask_lo) | k.magic) + czlo;
  out[1] = as_half2((w & k.mask_hi) | k.magic) * sixteenth + czhi;
  out[2] = as_half2((w8 & k.mask_lo) | k.magic) + czlo;
  out[3] = as_half2((w8 & k.mask_hi) | k.magic) * sixteenth + czhi;
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
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform: keeps tile/K-range math scalar
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

  // ---- activation slab [M][KR] -> LDS, each 8-block in K order 0,4,1,5,2,6,3,7.  The
  // global loads are issued before the weight loads: memory returns in issue order, so the
  // slab (L2 hits) must not queue behind the HBM stream it is needed to consume.
  constexpr int kSlabLoads = 2;  // 16-byte activation loads per thread kept in flight
  const int kb_per_row = KR >> 3;
  const int slab_items = p.M * kb_per_row;
  const uint16_t* xs = (const uint16_t*)p.x;
  uint4_t xv[kSlabLoads];
#pragma unroll
  for (int u = 0; u < kSlabLoads; ++u) {
    const int idx = tid + u * nthreads;
    if (idx < slab_items) {
      const int m = idx / kb_per_row;
      const int kb = idx - m * kb_per_row;
      xv[u] = *(const uint4_t*)(xs + (size_t)m * p.K + kwg0 + kb * 8);
    }
  }
  auto store_slab = [&](int idx, uint4_t v) {
    const int m = idx / kb_per_row;
    const int kb = idx - m * kb_per_row;
    uint4_t o;
    o.x = (v.x & 0xFFFFu) | (v.z << 16);
    o.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
    o.z = (v.y & 0xFFFFu) | (v.w << 16);
    o.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
    *(uint4_t*)(smem + (size_t)m * gp.slab_stride + kb * 16) = o;
  };

  // ---- issue the first kPrefetch chunks of weight loads before anything else
  // Addresses are a wave-uniform 64-bit base (scalar registers, advanced per step) plus a
  // per-lane 32-bit byte offset, so the loads use the scalar-base addressing mode and the
  // VALU does no address arithmetic in the loop.
  const char* wbase = (const char*)(p.qweight + (size_t)(kw0 / 8) * N);
  const uint32_t w_lane = ((uint32_t)kq * (uint32_t)N + (uint32_t)nl) * 4u;
  const size_t step_bytes = (size_t)N * 16;  // four packed rows
  const uint32_t s_lane = (uint32_t)nl * 2u;
  const uint32_t z_lane = (uint32_t)(nl >> 3) * 4u;
  const int zshift = (nl & 4) * 4;
  uint4_t wq[kPrefetch][kChunkSteps];
  uint2_t sc[kPrefetch][GPC];
  uint32_t zw[kPrefetch][GPC];
  auto load_chunk = [&](int c, uint4_t (&w)[kChunkSteps], uint2_t (&s)[GPC], uint32_t (&z)[GPC]) {
#pragma unroll
    for (int st = 0; st < kChunkSteps; ++st)
      w[st] = __builtin_nontemporal_load(
          (const uint4_t*)(wbase + (size_t)(c * kChunkSteps + st) * step_bytes + w_lane));
#pragma unroll
    for (int g = 0; g < GPC; ++g) {
      int gi = (kw0 + c * kChunkRows + g * GSTEPS * 32) / p.groupsize;
      gi = min(gi, p.num_groups - 1);
      s[g] = *(const uint2_t*)((const char*)p.scales + (size_t)gi * N * 2 + s_lane);
      z[g] = *(const uint32_t*)((const char*)p.qzeros + (size_t)gi * (N >> 3) * 4 + z_lane);
    }
  };
#pragma unroll
  for (int b = 0; b < kPrefetch; ++b)
    if (b < nchunks) load_chunk(b, wq[b], sc[b], zw[b]);

#pragma unroll
  for (int u = 0; u < kSlabLoads; ++u) {
    const int idx = tid + u * nthreads;
    if (idx < slab_items) store_slab(idx, xv[u]);
  }
  for (int idx = tid + kSlabLoads * nthreads; idx < slab_items; idx += nthreads) {
    const int m = idx / kb_per_row;
    const int kb = idx - m * kb_per_row;
    store_slab(idx, *(const uint4_t*)(xs + (size_t)m * p.K + kwg0 + kb * 8));
  }
  __syncthreads();

  const bool row_live = j < p.M;  // A-operand row of this lane
  const unsigned char* a_base = smem + (size_t)j * gp.slab_stride + (size_t)(wkk * KW + kq * 8) * 2;

  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  float4_t tot[4] = {zero4, zero4, zero4, zero4};
  float4_t acc[4] = {zero4, zero4, zero4, zero4};
  half2_t czlo[4], czhi[4];
  const SpliceConsts splice = splice_consts();

  auto process_chunk = [&](int c, const uint4_t (&w)[kChunkSteps], const uint2_t (&s)[GPC],
                           const uint32_t (&z)[GPC]) {
    const int kc = kw0 + c * kChunkRows;
    bool group_start = true, group_end = true;
    if constexpr (!STATIC128 && GSTEPS == kChunkSteps) {
      group_start = (c == 0) || (kc % p.groupsize == 0);
      group_end = (c == nchunks - 1) || ((kc + kChunkRows) % p.groupsize == 0);
    }
#pragma unroll
    for (int st = 0; st < kChunkSteps; ++st) {
      const int gi = st / GSTEPS;
      const bool first = (st % GSTEPS) == 0;
      const bool last = (st % GSTEPS) == GSTEPS - 1;
      constexpr bool kStaticGroups = STATIC128 || GSTEPS != kChunkSteps;
      if (first && (kStaticGroups || group_start)) {
        // zero-point constants of the group: z = (stored + 1) & 15 per column
        const uint32_t z4 = gptq_zero_plus_one(z[gi]) >> zshift;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const uint32_t zz = (z4 >> (4 * t)) & 0xFu;
          czlo[t] = as_half2(0xE400E400u | zz | (zz << 16));        // -(1024 + z)
          czhi[t] = as_half2(0xD400D400u | (zz << 4) | (zz << 20));  // -(64 + z)
        }
      }
      uint4_t a = {0u, 0u, 0u, 0u};
      if (row_live) a = *(const uint4_t*)(a_base + (size_t)(c * kChunkRows + st * 32) * 2);
      const uint32_t words[4] = {w[st].x, w[st].y, w[st].z, w[st].w};
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        half2_t b[4];
        unpack_word_f16(words[t], czlo[t], czhi[t], splice, b);
        if (first && kStaticGroups) {
          acc[t] = mfma16<DTYPE>(a, b, zero4);
        } else {
          if (first && group_start) acc[t] = zero4;
          acc[t] = mfma16<DTYPE>(a, b, acc[t]);
        }
      }
      if (last && (kStaticGroups || group_end)) {
        const half2_t s01 = as_half2(s[gi].x), s23 = as_half2(s[gi].y);
        const float sf[4] = {(float)s01.x, (float)s01.y, (float)s23.x, (float)s23.y};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
#pragma unroll
          for (int r = 0; r < RMAX; ++r) tot[t][r] = fmaf(sf[t], acc[t][r], tot[t][r]);
        }
      }
    }
  };

  // ring of kPrefetch chunk buffers: consume slot b, then refill it with chunk c + kPrefetch
  for (int c0 = 0; c0 < nchunks; c0 += kPrefetch) {
#pragma unroll
    for (int b = 0; b < kPrefetch; ++b) {
      const int c = c0 + b;
      if (c < nchunks) {
        process_chunk(c, wq[b], sc[b], zw[b]);
        if (c + kPrefetch < nchunks) load_chunk(c + kPrefetch, wq[b], sc[b], zw[b]);
      }
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

  // ---- cross-workgroup split-K: write the partial, take a ticket, last one reduces.
  // Partials and the ticket move with agent-scope relaxed atomics (coherent loads/stores
  // that bypass the per-XCD L2 state) instead of release/acquire fences: a fence here
  // would write back and invalidate the whole L2 once per workgroup, which costs more
  // than the kernel itself.  Ordering comes from waiting for the stores to be
  // acknowledged (vmcnt(0)) before the workgroup barrier that precedes the ticket.
  if (wkk == 0) {
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      const int m = 4 * kq + r;
      if (m < p.M) {
        float* dst = gp.partials + ((size_t)split * p.M + m) * N + nl;
#pragma unroll
        for (int t = 0; t < 4; ++t)
          __hip_atomic_store(dst + t, tot[t][r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  __shared__ uint32_t ticket_s;
  if (tid == 0) {
    ticket_s = __hip_atomic_fetch_add(gp.tickets + tile, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (ticket_s != (uint32_t)(gp.splits - 1)) return;
  {
    const int items = p.M * tile_cols;
    const int nbase = tile * tile_cols;
    for (int idx = tid; idx < items; idx += nthreads) {
      const int m = idx / tile_cols;
      const int n = nbase + (idx - m * tile_cols);
      const float* src = gp.partials + (size_t)m * N + n;
      const size_t sstride = (size_t)p.M * N;
      float sum = 0.f;
      int sp = 0;
      for (; sp + 8 <= gp.splits; sp += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          v[u] = __hip_atomic_load(src + (size_t)(sp + u) * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += v[u];
      }
      for (; sp < gp.splits; ++sp)
        sum += __hip_atomic_load(src + (size_t)sp * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      y[(size_t)m * N + n] = finish_output<DTYPE>(sum, p.bias, n);
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
  // Measured on MI355X (Llama-3-8B shapes, M=1): 64-column tiles with 4 waves along K per
  // workgroup and about two workgroups per CU (512 in flight) is the best point; wider
  // workgroups start too slowly and more splits lengthen the reduction tail.  The
  // activation slab (M rows x K/splits) must fit 60 KB of LDS.
  GemvConfig c;
  const int chunks = w->K / 128;
  c.wcol = 1;
  c.wk = chunks % 4 == 0 ? 4 : (chunks % 2 == 0 ? 2 : 1);
  const int per_wg = chunks / c.wk;  // chunks left to distribute over splits x per-wave work
  const int ntiles = w->N / 64;
  const int target_wgs = M <= 4 ? 512 : 384;  // partial-sum traffic grows with M
  int want = (target_wgs + ntiles / 2) / ntiles;
  if (want < 1) want = 1;
  const long lds_budget = 60000 - 16L * M;
  int min_splits = (int)(((long)M * w->K * 2 + lds_budget - 1) / lds_budget);
  if (min_splits < 1) min_splits = 1;
  int best = per_wg;  // always legal: one chunk per wave
  long best_cost = -1;
  for (int d = 1; d <= per_wg; ++d) {
    if (per_wg % d != 0 || d < min_splits) continue;
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
