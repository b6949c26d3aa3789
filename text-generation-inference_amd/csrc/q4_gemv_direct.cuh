// Decode kernel for the GPTQ layout with contiguous groups, up to 16 activation rows: the
// short-launch variant.
//
// A decode launch over a small projection (4096 x 4096: 8.4 MB) lives for a few microseconds,
// and what it does before its first weight load is out and after its last one has arrived is
// most of what separates it from a kernel that only reads.  This kernel keeps both ends short:
//   * The work decomposition is the grid itself (blockIdx.x = column tile of 64, blockIdx.y =
//     K split); the 128-row chunks are dealt to the splits x waves slots in order, the first
//     `rem` slots one more than the others, so a wave finds its range with a multiply and a
//     minimum: no division, a parameter block of about 100 bytes.
//   * No activation slab and no barrier before the first MFMA.  Up to four rows a wave fetches
//     the 128-row chunk of all its rows with one 16-byte load per lane and passes it through 1 KB
//     of LDS of its own into operand order; beyond, the lanes whose MFMA row is a live
//     activation row fetch 16 bytes of x per 32-row step straight from global memory (x stays
//     in L2).  Either way the loads are issued ahead of the weight words they meet, and one byte
//     permute per register puts them in the K order of the nibble splice.
//   * The arithmetic is that of gemv_gptq_lean_kernel: spliced nibbles enter the MFMA with
//     their offsets (1024 + q / 64 + q; bf16: 128 + q), one more MFMA per step against a
//     constant B operand gives P = sum x_k c_k and S = sum x_k, and a chunk contributes
//     scale * (acc - P - z * S) in fp32.
//   * One barrier at the end: every K wave leaves its 64 x M sums in LDS and they are added with
//     lane l owning column l.  K split across workgroups: fp16 rows take one 64-bit fixed-point
//     atomic per output element (the workgroup that completes a cell writes y and clears it:
//     cell_increment / cell_value in q4_gemv_kernels.cuh) while their cells fit the workspace;
//     bf16 and wider outputs write fp32 partial sums, draw a ticket per column tile, and the last
//     workgroup adds the partials in split order (what that sequence relies on is described at
//     gemv_finish).  One memory round trip against three: at 16 rows the ticket combine cost
//     3.5 us of a 9 us launch on 4096 x 4096, the cells 1.3 us.
#pragma once
#include "q4_gemv_lean.cuh"

namespace q4 {

struct DirectParams {
  const uint32_t* __restrict__ qweight;
  const uint32_t* __restrict__ qzeros;
  const half_t* __restrict__ scales;
  const void* __restrict__ x;
  const void* __restrict__ bias;
  void* __restrict__ y;
  unsigned long long* __restrict__ cells;  // [M][N] accumulation cells, zero between launches, or nullptr
  float* __restrict__ partials;            // [splits][M][N] partial sums (ticket combine), or nullptr
  uint32_t* __restrict__ tickets;          // one per column tile, zero between launches
  int N, K, M;
  int cpw;         // 128-row chunks per (split, wave) slot ...
  int rem;         // ... the first `rem` slots walk one more
  int gshift;      // group of chunk c = min(c >> gshift, num_groups - 1)
  int num_groups;
  int splits;
#ifdef Q4_PHASE_STAMPS
  unsigned long long* __restrict__ stamps;
#endif
};

// MR: activation rows padded to 1, 2, 4 or 16.  Up to four rows sit in the first register quad
// of the MFMA result (lanes of K block 0); sixteen fill it (lane block kq holds rows 4 kq .. 4 kq + 3).
// LOOP: some wave walks four chunks or more (the K loop proper); without it a wave has one to
// three chunks and the kernel is straight-line code with fewer registers.
template <int DTYPE, int MR, bool LOOP>
__global__ __launch_bounds__(512) void gemv_gptq_direct_kernel(DirectParams dp) {
  static_assert(MR == 1 || MR == 2 || MR == 4 || MR == 16, "rows are padded to 1, 2, 4 or 16");
  extern __shared__ __align__(16) unsigned char smem[];
  PhaseStamps ps;
  constexpr int RL = MR < 4 ? MR : 4;  // live rows among a lane's four
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wk = blockDim.x >> 6;
  const int j = lane & 15, kq = lane >> 4;
  const int N = dp.N;
  const int col = blockIdx.x * 64 + 4 * j;  // lane's first column
  const int slot = blockIdx.y * wk + wave;
  const int c0 = slot * dp.cpw + min(slot, dp.rem);
  const int nchunks = dp.cpw + (slot < dp.rem ? 1 : 0);
  constexpr int PF = 2;  // chunks of loads in flight per wave

  // Buffer loads: a scalar descriptor, one constant 32-bit lane offset and a scalar offset that
  // moves (no 64-bit vector address arithmetic).  Ranges are checked on the host.
  const direct_rsrc_t wrsrc = direct_rsrc(dp.qweight, (uint32_t)(dp.K >> 3) * (uint32_t)N * 4u);
  const direct_rsrc_t srsrc = direct_rsrc(dp.scales, (uint32_t)dp.num_groups * (uint32_t)N * 2u);
  const direct_rsrc_t zrsrc = direct_rsrc(dp.qzeros, (uint32_t)dp.num_groups * (uint32_t)(N >> 3) * 4u);
  const direct_rsrc_t xrsrc = direct_rsrc(dp.x, (uint32_t)dp.M * (uint32_t)dp.K * 2u);
  const uint32_t w_lane = ((uint32_t)kq * (uint32_t)N + (uint32_t)col) * 4u;
  const uint32_t s_lane = (uint32_t)col * 2u;
  const uint32_t z_lane = (uint32_t)(col >> 3) * 4u;
  const int zshift = (col & 7) * 4;
  const bool row_live = j < dp.M;  // this lane's MFMA row carries an activation row
  // (a row beyond M is beyond the end of x: the buffer load returns zeros without a memory access)
  const uint32_t x_lane = ((uint32_t)j * (uint32_t)dp.K + (uint32_t)kq * 8u) * 2u;
  const uint32_t step_bytes = (uint32_t)N * 16u;  // four packed rows

  // Up to four rows: the whole 128-row chunk of all of them is 4 x 256 bytes, one 16-byte load
  // per lane (lane l: row l / 16, bytes 16 (l % 16) ..); the wave passes it through its own 1 KB
  // of LDS into MFMA operand order.  Sixteen rows: every lane fetches the 16 bytes of its (row,
  // K block) per 32-row step itself.
  constexpr bool XLDS = MR <= 4;
  constexpr int XREGS = XLDS ? 1 : kChunkSteps;
  const uint32_t xl_lane = ((uint32_t)(lane >> 4) * (uint32_t)dp.K + (uint32_t)(lane & 15) * 8u) * 2u;
  unsigned char* xbuf = smem + wave * 1024;  // this wave's activation chunk (XLDS)
  struct Chunk {
    uint4_t x[XREGS];
    uint4_t w[kChunkSteps];
    uint2_t s;
    uint32_t z;
  };
  Chunk qa, qb;  // the ring: two chunks of loads in flight
  // No load of the K loop sits behind a branch: an activation row past M lies past the end of x
  // (such a buffer load returns zeros and touches no memory), one to three chunks per wave are
  // straight-line code, and the loop variant issues its refills unconditionally, the ones past
  // the wave's range out of bounds.  With a branch around a load the compiler cannot count the
  // loads in flight and waits for all of them, the newest chunk included, before it touches
  // the oldest (measured: one memory round trip per chunk, 1.25 us, whatever the ring holds).
  auto load_chunk = [&](int c, Chunk& q) {
    const uint32_t chunk = (uint32_t)(c0 + c);
    // loop variant: a chunk past the wave's range gets bit 31 into its lane offsets, which puts
    // it past the end of every tensor (the host keeps them below 2 GB there): zeros, no access
    const uint32_t past = LOOP && c >= nchunks ? 0x80000000u : 0u;
    // activations first: memory returns in issue order, and an L2 hit must not queue behind
    // the weight stream of this wave
    if constexpr (XLDS) {
      q.x[0] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, xl_lane | past, chunk * (kChunkRows * 2u), 0));
    } else {
#pragma unroll
      for (int st = 0; st < kChunkSteps; ++st)
        q.x[st] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, x_lane | past, (chunk * kChunkRows + st * 32) * 2u, 0));
    }
#pragma unroll
    for (int st = 0; st < kChunkSteps; ++st)
      q.w[st] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, w_lane | past, (chunk * kChunkSteps + st) * step_bytes, 2));
    // scale and zero point are needed when the chunk's last MFMA is done: asked for behind the
    // weights, they arrive with them instead of holding their return back
    const uint32_t gi = (uint32_t)min((int)(chunk >> dp.gshift), dp.num_groups - 1);
    q.s = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(srsrc, s_lane | past, gi * (uint32_t)N * 2u, 0));
    q.z = __builtin_amdgcn_raw_buffer_load_b32(zrsrc, z_lane | past, gi * (uint32_t)(N >> 3) * 4u, 0);
  };

  // constant B operand: column 0 the splice offsets c_k, column 1 ones
  uint4_t bconst = {0u, 0u, 0u, 0u};
  if (j == 0) bconst = uint4_t{LeanSplice<DTYPE>::kOffLo, LeanSplice<DTYPE>::kOffHi, LeanSplice<DTYPE>::kOffLo, LeanSplice<DTYPE>::kOffHi};
  if (j == 1) bconst = uint4_t{LeanSplice<DTYPE>::kOnes, LeanSplice<DTYPE>::kOnes, LeanSplice<DTYPE>::kOnes, LeanSplice<DTYPE>::kOnes};
  const LeanConsts kc = lean_consts<DTYPE>();
  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  const int row_lane0 = lane & 48;  // first lane of this lane's row of 16
  float tot[4][RL];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int i = 0; i < RL; ++i) tot[t][i] = 0.f;
  bool poisoned = false;  // some chunk of this wave met an inf or NaN activation

  // 16 bytes of activations into the K order [0,4,1,5,2,6,3,7] of the splice
  auto k_order = [](const uint4_t v) {
    uint4_t a;
    a.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
    a.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
    a.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
    a.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
    return a;
  };
  auto process_chunk = [&](const Chunk& q) {
    // (scheduling fences around a chunk: without them the copies of this block in the schedule
    // below are interleaved with each other and the register count doubles)
    __builtin_amdgcn_sched_barrier(0);
    float4_t acc[4], accc;
    if constexpr (XLDS) *(uint4_t*)(xbuf + lane * 16) = k_order(q.x[0]);  // rows beyond M: zeros
#pragma unroll
    for (int st = 0; st < kChunkSteps; ++st) {
      uint4_t a = {0u, 0u, 0u, 0u};
      if constexpr (XLDS) {
        if (j < 4) a = *(const uint4_t*)(xbuf + j * 256 + (st * 4 + kq) * 16);
      } else {
        a = k_order(q.x[st]);
      }
      const uint32_t words[4] = {q.w[st].x, q.w[st].y, q.w[st].z, q.w[st].w};
#pragma unroll
      for (int t = 0; t < 4; ++t) acc[t] = lean_mfma<DTYPE>(a, lean_unpack<DTYPE>(words[t], kc), st == 0 ? zero4 : acc[t]);
      accc = lean_mfma<DTYPE>(a, bconst, st == 0 ? zero4 : accc);
    }
    // scale * (acc - P - z * S); P and S of a row sit in columns 0 and 1 of the constant product
    const uint32_t z4 = gptq_zero_plus_one(q.z) >> zshift;
    float sf[4], zf[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      const half2_t sp = as_half2(t < 2 ? q.s.x : q.s.y);
      sf[t] = (float)((t & 1) ? sp.y : sp.x);
      zf[t] = (float)((z4 >> (4 * t)) & 0xFu);
    }
#pragma unroll
    for (int i = 0; i < RL; ++i) {
      // (a copy first: __builtin_bit_cast of a vector element reads element 0 whatever the index)
      const float ci = accc[i];
      float P, S;
      if constexpr (MR <= 4) {  // the rows sit in lane block 0: wave-uniform values
        P = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ci), 0));
        S = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, ci), 1));
      } else {
        P = row_lane(ci, row_lane0);
        S = row_lane(ci, row_lane0 + 1);
      }
      poisoned |= !(fabsf(S) <= 3.0e38f);  // an inf or NaN activation in this row's chunk
#pragma unroll
      for (int t = 0; t < 4; ++t) tot[t][i] = fmaf(sf[t], acc[t][i] - fmaf(zf[t], S, P), tot[t][i]);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // The wave's chunks, two in flight.  One, two and three chunks are straight-line code (a
  // kernel variant of its own: 88-120 registers); from four on a loop whose refills are
  // unconditional.  Either way every wait can be counted at compile time.
  static_assert(PF == 2, "the schedule below is written for two chunks in flight");
  // chunks c (in qa), c + 1 (in qb) and, with three left, c + 2
  auto end_piece = [&](int c, bool three, bool first) {
    process_chunk(qa);
    if (first) ps.mark_after(2, tot[0][0]);
    if (three) {
      load_chunk(c + 2, qa);
      process_chunk(qb);
      process_chunk(qa);
    } else {
      process_chunk(qb);
    }
  };
  if (nchunks == 1) {
    load_chunk(0, qa);
    ps.mark(6);
    ps.mark(1);
    process_chunk(qa);
    ps.mark_after(2, tot[0][0]);
  } else if (nchunks <= 3) {
    load_chunk(0, qa);
    load_chunk(1, qb);
    ps.mark(6);
    ps.mark(1);
    end_piece(0, nchunks == 3, true);
  } else if constexpr (LOOP) {
    load_chunk(0, qa);
    load_chunk(1, qb);
    ps.mark(6);
    ps.mark(1);
    for (int c = 0; c < nchunks; c += 2) {
      process_chunk(qa);
      if (c == 0) ps.mark_after(2, tot[0][0]);
      load_chunk(c + 2, qa);
      if (c + 1 < nchunks) process_chunk(qb);
      load_chunk(c + 3, qb);
    }
  }
  ps.mark_after(3, tot[0][0]);

  // A row with an infinite activation: acc, P and S are all infinite and their difference is NaN,
  // where the dot product with the dequantized weights is +-inf.  A wave that met one (rare)
  // walks its K range again, step by step, with the zero point taken out of the weights before
  // the MFMA: the class of every output is then that of fp32 arithmetic on s * (q - z).
  if (__builtin_amdgcn_ballot_w64(poisoned) != 0ull) {
    const SpliceConsts splice = splice_consts();
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < RL; ++i) tot[t][i] = 0.f;
    for (int c = 0; c < nchunks; ++c) {
      const uint32_t chunk = (uint32_t)(c0 + c);
      const uint32_t gi = (uint32_t)min((int)(chunk >> dp.gshift), dp.num_groups - 1);
      const uint2_t sv = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(srsrc, s_lane, gi * (uint32_t)N * 2u, 0));
      const uint32_t z4 = gptq_zero_plus_one(__builtin_amdgcn_raw_buffer_load_b32(zrsrc, z_lane, gi * (uint32_t)(N >> 3) * 4u, 0)) >> zshift;
      half2_t czlo[4], czhi[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const uint32_t zz = (z4 >> (4 * t)) & 0xFu;
        czlo[t] = as_half2(0xE400E400u | zz | (zz << 16));         // -(1024 + z)
        czhi[t] = as_half2(0xD400D400u | (zz << 4) | (zz << 20));  // -(64 + z)
      }
      float4_t ex[4] = {zero4, zero4, zero4, zero4};
      for (int st = 0; st < kChunkSteps; ++st) {
        uint4_t xv = {0u, 0u, 0u, 0u};
        if (row_live)
          xv = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, x_lane, (chunk * kChunkRows + st * 32) * 2u, 0));
        const uint4_t wv = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(wrsrc, w_lane, (chunk * kChunkSteps + st) * step_bytes, 0));
        uint4_t a;
        a.x = __builtin_amdgcn_perm(xv.z, xv.x, 0x05040100u);
        a.y = __builtin_amdgcn_perm(xv.z, xv.x, 0x07060302u);
        a.z = __builtin_amdgcn_perm(xv.w, xv.y, 0x05040100u);
        a.w = __builtin_amdgcn_perm(xv.w, xv.y, 0x07060302u);
        const uint32_t words[4] = {wv.x, wv.y, wv.z, wv.w};
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          half2_t b[4];
          unpack_word_f16(words[t], czlo[t], czhi[t], splice, b);
          ex[t] = mfma16<DTYPE>(a, b, ex[t]);
        }
      }
#pragma unroll
      for (int t = 0; t < 4; ++t) {
        const half2_t sp = as_half2(t < 2 ? sv.x : sv.y);
        const float sf = (float)((t & 1) ? sp.y : sp.x);
#pragma unroll
        for (int i = 0; i < RL; ++i) tot[t][i] = fmaf(sf, ex[t][i], tot[t][i]);
      }
    }
  }

  // ---- the K waves meet in LDS: wave w leaves row r at red[(w * MR + r) * 64 + column]
  float* red = (float*)(smem + (XLDS ? wk * 1024 : 0));
  if (MR == 16 || kq == 0) {
#pragma unroll
    for (int i = 0; i < RL; ++i) {
      const int r = (MR == 16 ? 4 * kq : 0) + i;
      *(float4_t*)(red + (wave * MR + r) * 64 + 4 * j) = float4_t{tot[0][i], tot[1][i], tot[2][i], tot[3][i]};
    }
  }
  if (wk > 1) __syncthreads();
  uint16_t* y = (uint16_t*)dp.y;
  const int n = blockIdx.x * 64 + lane;
  auto row_sum = [&](int r) {
    float v = red[r * 64 + lane];
    for (int w = 1; w < wk; ++w) v += red[(w * MR + r) * 64 + lane];
    return v;
  };

  if (dp.cells != nullptr && MR >= 2 && dp.M > 1) {
    // one 64-bit fixed-point atomic per element; the rows are dealt to the waves, two adds of a
    // wave in flight at a time (from two rows on: wave 0 taking the rows in turn pays one round
    // trip per row, 0.4-0.9 us per launch and row on the Llama-3-8B projections)
    for (int r0 = wave; r0 < dp.M; r0 += 2 * wk) {
      const int r1 = r0 + wk;
      const bool two = r1 < dp.M;
      const float v0 = row_sum(r0);
      const float v1 = two ? row_sum(r1) : 0.f;
      if (r0 == wave) ps.mark_after(4, v0);
      unsigned long long* cell0 = dp.cells + (size_t)r0 * N + n;
      unsigned long long* cell1 = dp.cells + (size_t)(two ? r1 : r0) * N + n;
      const unsigned long long inc0 = cell_increment(v0), inc1 = cell_increment(v1);
      unsigned long long before0, before1 = 0ull;
      before0 = __hip_atomic_fetch_add(cell0, inc0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      if (two) before1 = __hip_atomic_fetch_add(cell1, inc1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      ps.mark_after(5, __builtin_bit_cast(float, (uint32_t)before0));
      const unsigned long long now0 = before0 + inc0, now1 = before1 + inc1;
      if (cell_complete(now0, dp.splits)) {
        y[(size_t)r0 * N + n] = finish_output<DTYPE>(cell_value(now0), dp.bias, n);
        __hip_atomic_store(cell0, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      if (two && cell_complete(now1, dp.splits)) {
        y[(size_t)r1 * N + n] = finish_output<DTYPE>(cell_value(now1), dp.bias, n);
        __hip_atomic_store(cell1, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  } else if (dp.cells != nullptr) {
    // a single row: one 64-bit fixed-point atomic per element from wave 0
    if (wave == 0) {
#pragma unroll
      for (int m = 0; m < RL; ++m) {
        if (m < dp.M) {
          const float v = row_sum(m);
          if (m == 0) ps.mark_after(4, v);
          unsigned long long* cell = dp.cells + (size_t)m * N + n;
          const unsigned long long inc = cell_increment(v);
          const unsigned long long before = __hip_atomic_fetch_add(cell, inc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          ps.mark_after(5, __builtin_bit_cast(float, (uint32_t)before));
          const unsigned long long now = before + inc;
          if (cell_complete(now, dp.splits)) {
            y[(size_t)m * N + n] = finish_output<DTYPE>(cell_value(now), dp.bias, n);
            __hip_atomic_store(cell, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          }
        }
      }
    }
  } else if (dp.splits == 1) {
    // the rows are dealt to the waves: wave w finishes rows w, w + wk, ..
    for (int r = wave; r < dp.M; r += wk) {
      const float v = row_sum(r);
      if (r == wave) ps.mark_after(4, v);
      y[(size_t)r * N + n] = finish_output<DTYPE>(v, dp.bias, n);
    }
  } else {
    // fp32 partial sums, a ticket per column tile, the last workgroup adds in split order
    for (int r = wave; r < dp.M; r += wk) {
      const float v = row_sum(r);
      if (r == wave) ps.mark_after(4, v);
      __hip_atomic_store(dp.partials + ((size_t)blockIdx.y * dp.M + r) * N + n, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    uint32_t* ticket_s = (uint32_t*)(red + wk * MR * 64);
    uint32_t* ticket = dp.tickets + blockIdx.x;
    if (threadIdx.x == 0) *ticket_s = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    ps.mark(5);
    if (*ticket_s == (uint32_t)(dp.splits - 1)) {
      const size_t sstride = (size_t)dp.M * N;
      for (int r = wave; r < dp.M; r += wk) {
        const float* src = dp.partials + (size_t)r * N + n;
        float sum = 0.f;
        int sp = 0;
        for (; sp + 8 <= dp.splits; sp += 8) {
          float v[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) v[u] = __hip_atomic_load(src + (size_t)(sp + u) * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
          for (int u = 0; u < 8; ++u) sum += v[u];
        }
        for (; sp < dp.splits; ++sp) sum += __hip_atomic_load(src + (size_t)sp * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        y[(size_t)r * N + n] = finish_output<DTYPE>(sum, dp.bias, n);
      }
      if (threadIdx.x == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
#ifdef Q4_PHASE_STAMPS
  ps.flush_to(dp.stamps, lane, wave);
#endif
}

}  // namespace q4
