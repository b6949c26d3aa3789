// Decode kernel for the GPTQ layout with contiguous groups of 128 rows (or a multiple), up to
// 16 activation rows per workgroup: the instruction-lean variant.
//
// Same streaming, tiling and split-K as gemv_gptq_kernel (q4_gemv_kernels.cuh); what changes is
// the arithmetic around the MFMA:
//   * The spliced nibbles go into the B operand as they are.  In fp16, nibbles 0,4,2,6 of a word
//     become 1024 + q (mantissa splice into 1024.0) and nibbles 1,5,3,7, which sit four bits
//     higher, become 64 + q (the same splice into 64.0, whose mantissa step is 1/16): four
//     v_and_or_b32 and one shift per packed word, no packed-half arithmetic at all.
//   * What the offsets and the zero point add to a group's sum does not depend on the weights:
//     sum_k x_k (c_k + q_k - (c_k + z)) with c_k in {1024, 64}.  One more MFMA per 32-row step
//     with a constant B operand (column 0: the c_k pattern, column 1: ones) accumulates
//     P = sum x_k c_k and S = sum x_k per activation row next to the real columns, and the
//     group's contribution becomes scale * (acc - P - z * S) in fp32.
//   * With few activation rows the sixteen rows of the MFMA are used for different groups:
//     the A operand of group g carries x in row (g mod GACC) of each activation row's block
//     and zeros elsewhere, so the per-group sums of GACC = 16 / MP consecutive groups pile up
//     in separate accumulator rows and scale / zero / correction are applied once per GACC
//     groups instead of once per group (one row: once per 2048 weights rows of K).
//   * bf16 activations: every nibble is shifted down and spliced into 128.0 (seven VALU
//     operations per word); the MFMA is the bf16 one, no fp16 -> bf16 conversion of weights.
// The dequantized weight a one-hot activation row reads back is still exactly
// round(scale * (q - z)): 1024 + q, P = 1024 and z * S = z are exact in fp32.
#pragma once
#include "q4_gemv_kernels.cuh"

namespace q4 {

template <int DTYPE>
struct LeanSplice {
  // fp16: low nibble of each half into 1024.0, the nibble above it into 64.0
  static constexpr uint32_t kMagicLo = DTYPE == Q4_DTYPE_F16 ? 0x64006400u : 0x43004300u;
  static constexpr uint32_t kMagicHi = DTYPE == Q4_DTYPE_F16 ? 0x54005400u : 0x43004300u;
  // offsets c_k of the eight K slots of a lane, in the splice order [0,4,1,5,2,6,3,7]
  static constexpr uint32_t kOffLo = DTYPE == Q4_DTYPE_F16 ? 0x64006400u : 0x43004300u;  // (1024, 1024) / (128, 128)
  static constexpr uint32_t kOffHi = DTYPE == Q4_DTYPE_F16 ? 0x54005400u : 0x43004300u;  // (64, 64) / (128, 128)
  static constexpr uint32_t kOnes = DTYPE == Q4_DTYPE_F16 ? 0x3C003C00u : 0x3F803F80u;
};

struct LeanConsts {
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};
template <int DTYPE>
__device__ __forceinline__ LeanConsts lean_consts() {
  LeanConsts k{0x000F000Fu, 0x00F000F0u, LeanSplice<DTYPE>::kMagicLo, LeanSplice<DTYPE>::kMagicHi};
  // register operands: the compiler then selects the fused v_and_or_b32 (see splice_consts)
  asm volatile("" : "+s"(k.mask_lo), "+s"(k.mask_hi), "+v"(k.magic_lo), "+v"(k.magic_hi));
  return k;
}

// Eight spliced weights of a packed word in K order [0,4,1,5,2,6,3,7]: c_k + q_k.
template <int DTYPE>
__device__ __forceinline__ uint4_t lean_unpack(uint32_t w, const LeanConsts& k) {
  uint4_t b;
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    const uint32_t w8 = w >> 8;
    b.x = (w & k.mask_lo) | k.magic_lo;
    b.y = (w & k.mask_hi) | k.magic_hi;
    b.z = (w8 & k.mask_lo) | k.magic_lo;
    b.w = (w8 & k.mask_hi) | k.magic_hi;
  } else {
    b.x = (w & k.mask_lo) | k.magic_lo;
    b.y = ((w >> 4) & k.mask_lo) | k.magic_lo;
    b.z = ((w >> 8) & k.mask_lo) | k.magic_lo;
    b.w = ((w >> 12) & k.mask_lo) | k.magic_lo;
  }
  return b;
}

template <int DTYPE>
__device__ __forceinline__ float4_t lean_mfma(const uint4_t a, const uint4_t b, float4_t c) {
  if constexpr (DTYPE == Q4_DTYPE_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// Value of lane `src` of the caller's row of 16 lanes.
__device__ __forceinline__ float row_lane(float v, int src_lane) {
  return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(src_lane << 2, __builtin_bit_cast(int, v)));
}

// MP: activation rows padded to a power of two (1, 2, 4, 8, 16).  GACC = 16 / MP chunks (groups
// of 128 rows) share one set of accumulators, one MFMA row per (activation row, chunk).
template <int DTYPE, int MP, int PF = 2>
__global__ __launch_bounds__(1024) void gemv_gptq_lean_kernel(GemvParams gp) {
  static_assert(MP == 1 || MP == 2 || MP == 4 || MP == 8 || MP == 16, "rows are padded to a power of two");
  static_assert(MP != 8 || PF % 2 == 0, "eight rows: the chunks of a ring round alternate between two accumulator rows");
  extern __shared__ __align__(16) unsigned char smem[];
  PhaseStamps ps;
  const Problem& p = gp.p;
  const Decomp d = make_decomp(gp, 64);
  const int N = p.N;
  const int nl = d.tile * d.tile_cols + d.wc * 64 + 4 * d.j;  // lane's first column
  const int nchunks = d.KW / kChunkRows;
  constexpr int GACC = 16 / MP;
  constexpr bool PER_CHUNK = MP >= 8;               // scale / zero applied after every chunk
  constexpr int NTOT = MP <= 4 ? 1 : MP / 4;        // activation rows among a lane's four MFMA rows
  constexpr int RMAX = MP == 1 ? 1 : (MP == 2 ? 2 : 4);

  const char* wbase = (const char*)(p.qweight + (size_t)(d.kw0 / 8) * N);
  const uint32_t w_lane = ((uint32_t)d.kq * (uint32_t)N + (uint32_t)nl) * 4u;
  const size_t step_bytes = (size_t)N * 16;  // four packed rows
  const uint32_t s_lane = (uint32_t)nl * 2u;
  const uint32_t z_lane = (uint32_t)(nl >> 3) * 4u;
  const int zshift = (nl & 7) * 4;
  struct Chunk { uint4_t w[kChunkSteps]; };
  struct Params { uint2_t s; uint32_t z; };  // four fp16 scales, the packed zero points of the lane's columns
  Chunk wq[PF];
  Params ring[PER_CHUNK ? PF : 1];
  auto load_params = [&](int c) {
    // group of chunk c of this wave (clamped: rows past the wave's range carry zero sums)
    int gi = (d.kw0 + min(c, nchunks - 1) * kChunkRows) / p.groupsize;
    gi = min(gi, p.num_groups - 1);
    Params r;
    r.s = *(const uint2_t*)((const char*)p.scales + (size_t)gi * N * 2 + s_lane);
    r.z = *(const uint32_t*)((const char*)p.qzeros + (size_t)gi * (N >> 3) * 4 + z_lane);
    return r;
  };
  auto load_chunk = [&](int c, Chunk& w) {
#pragma unroll
    for (int st = 0; st < kChunkSteps; ++st)
      w.w[st] = __builtin_nontemporal_load((const uint4_t*)(wbase + (size_t)(c * kChunkSteps + st) * step_bytes + w_lane));
  };
  // Period parameters (MP <= 4): scales and zero points of the four chunks whose sums sit in
  // this lane's accumulator rows.  They are asked for right behind the last weight loads of
  // the period: memory returns in issue order, so they arrive with the data they scale and
  // the (scattered, small) requests stay out of the way of the stream until then.
  Params per[PER_CHUNK ? 1 : 4];
  auto load_period = [&](int c_first) {
    if constexpr (!PER_CHUNK) {
#pragma unroll
      for (int r = 0; r < 4; ++r) per[r] = load_params(c_first + (4 * d.kq + r) % GACC);
    }
  };
  // cl: chunk whose loads were just issued; c_done: last chunk already processed.  A period
  // shorter than the ring is asked for when the period before it has been applied instead.
  auto period_after_chunk_load = [&](int cl, int c_done) {
    if constexpr (!PER_CHUNK) {
      if ((cl % GACC == GACC - 1 || cl == nchunks - 1) && cl - cl % GACC <= c_done + 1) load_period(cl - cl % GACC);
    }
  };
  auto issue_first_chunks = [&]() {
#pragma unroll
    for (int b = 0; b < PF; ++b)
      if (b < nchunks) {
        load_chunk(b, wq[b]);
        if constexpr (PER_CHUNK) ring[b] = load_params(b);
        period_after_chunk_load(b, -1);
      }
  };

  // ---- activations.  Every wave stages the K range it walks itself into its own piece of LDS
  // (rows x KW halves, each 8-block in the K order [0,4,1,5,2,6,3,7] of the splice): no wave
  // waits for another one, there is no workgroup barrier before the first MFMA.
  // (With several column waves per workgroup and many rows the pieces would not fit: the host
  // then asks for one slab per workgroup, staged by all waves and fenced by a barrier.)
  const int wstride = gp.slab_stride;  // bytes between activation rows of a wave's piece
  unsigned char* wslab = smem + (size_t)d.wave * gp.rows_per_block_alloc * wstride;
  if (!gp.wave_slab) {
    SlabStager<true, (MP == 16 ? 8 : 4)> slab;
    slab.issue(gp, d);
    issue_first_chunks();
    ps.mark(6);
    slab.store(gp, d, smem);
    wslab = smem + (size_t)d.kwo * 2;
  } else {
    const int kbw = d.KW >> 3;  // 16-byte blocks per row
    const uint16_t* xs = (const uint16_t*)p.x + (size_t)d.mb * p.K + (p.x_perm != nullptr ? 0 : d.kw0);
    const int32_t* cols = p.x_perm != nullptr ? p.x_perm + d.kw0 : nullptr;
    auto fetch = [&](int m, int kb) {
      const uint16_t* row = xs + (size_t)m * p.K;
      if (cols != nullptr) {
        // eight scattered columns of the row (it stays in L2); a bad index is clamped
        const uint4_t p0 = *(const uint4_t*)(cols + kb * 8);
        const uint4_t p1 = *(const uint4_t*)(cols + kb * 8 + 4);
        const int last = p.K - 1;
        auto at = [&](uint32_t i) { return (uint32_t)row[min(max((int)i, 0), last)]; };
        uint4_t o;
        o.x = at(p0.x) | (at(p0.y) << 16);
        o.y = at(p0.z) | (at(p0.w) << 16);
        o.z = at(p1.x) | (at(p1.y) << 16);
        o.w = at(p1.z) | (at(p1.w) << 16);
        return o;
      }
      return *(const uint4_t*)(row + kb * 8);
    };
    auto put = [&](int m, int kb, uint4_t v) {
      uint4_t o;
      o.x = (v.x & 0xFFFFu) | (v.z << 16);
      o.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
      o.z = (v.y & 0xFFFFu) | (v.w << 16);
      o.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
      *(uint4_t*)(wslab + (size_t)m * wstride + kb * 16) = o;
    };
    // The first batch of activation loads goes out before the weight loads: memory returns in
    // issue order, and the activations (L2 hits for all but the first workgroups) must not
    // queue behind two chunks of the HBM stream that the first MFMA does not need.
    constexpr int XB = MP >= 4 ? 4 : MP;  // rows whose loads are in flight together
    uint4_t x0[XB];
#pragma unroll
    for (int u = 0; u < XB; ++u)
      if (u < d.mloc && d.lane < kbw) x0[u] = fetch(u, d.lane);
    issue_first_chunks();
    ps.mark(6);
#pragma unroll
    for (int u = 0; u < XB; ++u)
      if (u < d.mloc && d.lane < kbw) put(u, d.lane, x0[u]);
    for (int kb = d.lane; kb < kbw; kb += 64) {
      for (int m0 = kb == d.lane ? XB : 0; m0 < d.mloc; m0 += XB) {
        uint4_t xv[XB];
#pragma unroll
        for (int u = 0; u < XB; ++u)
          if (m0 + u < d.mloc) xv[u] = fetch(m0 + u, kb);
#pragma unroll
        for (int u = 0; u < XB; ++u)
          if (m0 + u < d.mloc) put(m0 + u, kb, xv[u]);
      }
    }
  }
  // a block of zeros behind the pieces: A operand of the lanes whose MFMA row is not fed.
  // Every wave writes it (same values) so that none depends on another.
  if (d.lane < 32) ((uint4_t*)(smem + gp.slab_bytes))[d.lane] = uint4_t{0u, 0u, 0u, 0u};
  if (!gp.wave_slab) __syncthreads();
  ps.mark(1);

  // MFMA row j of this lane's A operand: activation row mj, chunk slot glj of the accumulators
  const int mj = d.j / GACC, glj = d.j % GACC;
  const bool row_ok = mj < d.mloc;
  const uint32_t a_real = (uint32_t)(wslab - smem) + (uint32_t)(mj * wstride + d.kq * 16);
  const uint32_t a_zero = (uint32_t)gp.slab_bytes;

  // constant B operand: column 0 the offsets c_k, column 1 ones
  uint4_t bconst = {0u, 0u, 0u, 0u};
  if (d.j == 0) bconst = uint4_t{LeanSplice<DTYPE>::kOffLo, LeanSplice<DTYPE>::kOffHi, LeanSplice<DTYPE>::kOffLo, LeanSplice<DTYPE>::kOffHi};
  if (d.j == 1) bconst = uint4_t{LeanSplice<DTYPE>::kOnes, LeanSplice<DTYPE>::kOnes, LeanSplice<DTYPE>::kOnes, LeanSplice<DTYPE>::kOnes};

  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  float4_t acc[4] = {zero4, zero4, zero4, zero4};
  float4_t accc = zero4;
  float tot[4][NTOT];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < NTOT; ++i) tot[t][i] = 0.f;
  const LeanConsts kc = lean_consts<DTYPE>();
  const int row_lane0 = d.lane & 48;  // first lane of this lane's row of 16

  // scale * (acc - P - z * S) of accumulator row r into tot[.][ti]
  auto apply = [&](const Params& pr, int r, int ti) {
    const float P = row_lane(accc[r], row_lane0);
    const float S = row_lane(accc[r], row_lane0 + 1);
    const uint32_t z4 = gptq_zero_plus_one(pr.z) >> zshift;
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const half2_t sp = as_half2(t < 2 ? pr.s.x : pr.s.y);
      const float sf = (float)((t & 1) ? sp.y : sp.x);
      const float zf = (float)((z4 >> (4 * t)) & 0xFu);
      tot[t][ti] = fmaf(sf, acc[t][r] - fmaf(zf, S, P), tot[t][ti]);
    }
  };

  auto process_chunk = [&](int c, int b, const Chunk& w) {
    // which MFMA rows this chunk feeds
    int u;
    if constexpr (MP == 16) u = 0;
    else if constexpr (MP == 8) u = b & 1;  // chunks come in pairs: PF is even
    else u = c % GACC;
    const bool live = row_ok && glj == u;
    const uint32_t a_addr = live ? a_real + (uint32_t)c * (kChunkRows * 2) : a_zero;
#pragma unroll
    for (int st = 0; st < kChunkSteps; ++st) {
      const uint4_t a = *(const uint4_t*)(smem + a_addr + st * 64);
      const uint32_t words[4] = {w.w[st].x, w.w[st].y, w.w[st].z, w.w[st].w};
      if (MP == 16 && st == 0) {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = lean_mfma<DTYPE>(a, lean_unpack<DTYPE>(words[t], kc), zero4);
        accc = lean_mfma<DTYPE>(a, bconst, zero4);
      } else {
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = lean_mfma<DTYPE>(a, lean_unpack<DTYPE>(words[t], kc), acc[t]);
        accc = lean_mfma<DTYPE>(a, bconst, accc);
      }
    }
    if constexpr (MP == 16) {
#pragma unroll
      for (int r = 0; r < 4; ++r) apply(ring[b], r, r);
    } else if constexpr (MP == 8) {
      // rows u and u + 2 of the lane (activation rows 2 kq and 2 kq + 1) are complete
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int r = u + 2 * h;
        apply(ring[b], r, h);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t][r] = 0.f;
        accc[r] = 0.f;
      }
    } else {
      if (u == GACC - 1 || c == nchunks - 1) {
#pragma unroll
        for (int r = 0; r < 4; ++r) apply(per[r], r, 0);
#pragma unroll
        for (int t = 0; t < 4; ++t) acc[t] = zero4;
        accc = zero4;
        // the next period's last loads are out already (it is shorter than the ring)
        if (c + 1 < nchunks && min(c + GACC, nchunks - 1) < c + PF) load_period(c + 1);
      }
    }
  };

  for (int c0 = 0; c0 < nchunks; c0 += PF) {
#pragma unroll
    for (int b = 0; b < PF; ++b) {
      const int c = c0 + b;
      if (c < nchunks) {
        process_chunk(c, b, wq[b]);
        if (c == 0) ps.mark_after(2, acc[0][0]);
        if (c + PF < nchunks) {
          load_chunk(c + PF, wq[b]);
          if constexpr (PER_CHUNK) ring[b] = load_params(c + PF);
          period_after_chunk_load(c + PF, c);
        }
      }
    }
  }

  ps.mark_after(3, tot[0][0]);
  // hand the sums to the common epilogue: slot r of lane (j, kq) is activation row 4 kq + r
  float out[4][RMAX];
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    if constexpr (MP == 1) {
      float v = tot[t][0];
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      out[t][0] = v;
    } else if constexpr (MP == 2) {
      float v = tot[t][0];
      v += __shfl_xor(v, 16, 64);  // lanes kq 0,1: row 0; kq 2,3: row 1
      out[t][0] = v;
      out[t][1] = __shfl(v, (d.lane & 15) + 32, 64);
    } else if constexpr (MP == 4) {
#pragma unroll
      for (int r = 0; r < 4; ++r) out[t][r] = __shfl(tot[t][0], (d.lane & 15) + 16 * r, 64);
    } else if constexpr (MP == 8) {
      // activation row 4 kq + r sits in lane row 2 kq + r / 2, slot r % 2 (only kq < 2 holds live rows)
#pragma unroll
      for (int r = 0; r < 4; ++r)
        out[t][r] = __shfl(tot[t][r & 1], ((d.lane & 15) + 16 * (2 * d.kq + (r >> 1))) & 63, 64);
    } else {
#pragma unroll
      for (int r = 0; r < 4; ++r) out[t][r] = tot[t][r];
    }
  }
  gemv_finish<DTYPE, 4, RMAX>(gp, d, out, nl, smem, ps);
}

}  // namespace q4
