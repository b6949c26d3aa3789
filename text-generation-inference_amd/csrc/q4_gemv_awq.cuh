// Decode kernel for the AWQ layout (qweight [K, N/8]: a word holds eight interleaved columns of
// one K row), up to 8 activation rows.
//
// The words go into the matrix core as they are stored; nothing is transposed.  A 16x16x16
// MFMA sums, per lane of its B operand, over four "K slots" -- and it does not care what the
// slots are as long as both operands agree.  Here the four slots of a lane are four COLUMNS of
// one K row (half a packed word after the nibble splice, which thanks to AWQ's interleave
// yields the columns in order), and the A operand is sparse: MFMA row 4 m + c carries x[m][k]
// in slot c and zeros in the other three.  Row 4 m + c of the result is then
// sum over the step's four K rows of x[m][k] * w[k][column c of the lane's half word]:
// a lane block kq of the accumulator holds activation row m = kq, its four registers four
// adjacent columns.  One MFMA serves four activation rows; rows 4..7 take a second A operand.
//
// Per packed word: the splice (four v_and_or_b32 and a shift in fp16) and two MFMAs.  Per
// K row and group of four activation rows: three operations for the A operand (the
// activation, fetched eight K rows at a time from the slab, is duplicated into both halves
// and masked into place).  As in the contiguous-group GPTQ kernel the spliced values keep their
// offsets (1024 + q or 64 + q; 128 + q in bf16): a group's sum is scale * (acc - (c + z) * S)
// with S the sum of the group's activations, which the lanes add up from the activation
// operands they fetch anyway.  The dequantized weight a one-hot activation row reads back is
// still exactly round(scale * (q - z)).
//
// Tiling, activation slab, K partition, split-K and the output stage are those of the other
// decode kernels: wave tile 256 columns (two words per lane) x 32 rows per step, lane (j, kq)
// loads rows 8 kq .. 8 kq + 7 of the step, 128-byte row segments per 16 lanes.
#pragma once
#include "q4_gemv_lean.cuh"

namespace q4 {

typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));

template <int DTYPE>
__device__ __forceinline__ float4_t diag_mfma(const uint2_t a, const uint2_t b, float4_t c) {
  if constexpr (DTYPE == Q4_DTYPE_F16)
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4_t, a), __builtin_bit_cast(half4_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(short4_t, a), __builtin_bit_cast(short4_t, b), c, 0, 0, 0);
}

// fp32 sum of the eight activations in v
template <int DTYPE>
__device__ __forceinline__ float sum8(const uint4_t v) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (DTYPE == Q4_DTYPE_F16) {
      const half2_t h = as_half2(w[i]);
      s += (float)h.x + (float)h.y;
    } else {
      s += __builtin_bit_cast(float, w[i] << 16) + __builtin_bit_cast(float, w[i] & 0xFFFF0000u);
    }
  }
  return s;
}

// G: groups of four activation rows (1 or 2: up to 8 rows; a four-group variant for 9-16 rows
// measured 25-35 % slower than the transposing kernel: 31 against 23 us for 4096 x 14336 at M = 9).
template <int DTYPE, int G>
__global__ __launch_bounds__(512) void gemv_awq_diag_kernel(GemvParams gp) {
  extern __shared__ __align__(16) unsigned char smem[];
  const Problem& p = gp.p;
  const Decomp d = make_decomp(gp, 256);
  const int N = p.N;
  const int NC = N >> 3;                                             // packed words per row
  const int cw = (d.tile * d.tile_cols + d.wc * 256) / 8 + 2 * d.j;  // first of this lane's 2 words
  const int col0 = cw * 8;
  const int nsteps = d.KW / 32;
  // 32-row steps (8 x 64-bit loads each) in flight per wave: one 128-row chunk.  A wave's K
  // range is whole chunks, so the first four steps are loaded unconditionally and the loop
  // refills a step's registers with the same step of the next chunk without a test; the last
  // chunk is processed outside the loop.  (With a branch around a load the compiler cannot count
  // the loads in flight: the activation staging below then waits for the whole weight prefetch
  // and every step for the newest refill.)
  constexpr int PF = 4;

  SlabStager<false> slab;
  slab.issue(gp, d, nullptr);

  const char* wbase = (const char*)(p.qweight + (size_t)d.kw0 * NC);
  const uint32_t w_lane = ((uint32_t)(d.kq * 8) * (uint32_t)NC + (uint32_t)cw) * 4u;
  const size_t row_bytes = (size_t)NC * 4;
  uint2_t wq[PF][8];
  auto load_step = [&](int st, uint2_t (&w)[8]) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      w[r] = __builtin_nontemporal_load((const uint2_t*)(wbase + (size_t)(st * 32 + r) * row_bytes + w_lane));
  };
#pragma unroll
  for (int b = 0; b < PF; ++b) load_step(b, wq[b]);

  // scales (16 halves) and zero points (2 words) of the lane's columns for one group: asked
  // for when the group starts, used when it ends
  struct GroupParams { uint4_t s0, s1; uint2_t z; };
  auto load_group = [&](int g) {
    GroupParams r;
    const uint4_t* sp = (const uint4_t*)(p.scales + (size_t)g * N + col0);
    r.s0 = sp[0];
    r.s1 = sp[1];
    r.z = *(const uint2_t*)(p.qzeros + (size_t)g * NC + cw);
    return r;
  };
  const int g_first = min(d.kw0 / p.groupsize, p.num_groups - 1);
  GroupParams gpar = load_group(g_first);

  slab.store(gp, d, smem);
  __syncthreads();

  // A operand: MFMA row j of this lane is (activation row 4 g + j / 4, slot j % 4)
  const int slot = d.j & 3;
  uint32_t amask0[G], amask1[G];
  uint32_t a_off[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const int m = 4 * g + (d.j >> 2);
    const bool live = m < d.mloc;
    const uint32_t half_mask = (slot & 1) ? 0xFFFF0000u : 0x0000FFFFu;
    amask0[g] = live && slot < 2 ? half_mask : 0u;
    amask1[g] = live && slot >= 2 ? half_mask : 0u;
    a_off[g] = (uint32_t)((live ? m : 0) * gp.slab_stride + (d.kwo + d.kq * 8) * 2);
  }
  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  float4_t acc[2][2][G];  // [word][half word][row group]
  float xsum[G];          // sum of this lane's activations (row 4 g + j / 4, K block kq) over the group so far
  float tot[16][G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    xsum[g] = 0.f;
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int h = 0; h < 2; ++h) acc[b][h][g] = zero4;
  }
#pragma unroll
  for (int t = 0; t < 16; ++t)
#pragma unroll
    for (int g = 0; g < G; ++g) tot[t][g] = 0.f;
  const LeanConsts kc = lean_consts<DTYPE>();
  const int row_lane0 = d.lane & 48;
  constexpr float kOffLo = DTYPE == Q4_DTYPE_F16 ? 1024.f : 128.f;
  constexpr float kOffHi = DTYPE == Q4_DTYPE_F16 ? 64.f : 128.f;

  // scale * (acc - (c + z) * S) of the finished group into tot; accumulators back to zero
  auto flush = [&](const GroupParams& gr) {
    const uint32_t su[8] = {gr.s0.x, gr.s0.y, gr.s0.z, gr.s0.w, gr.s1.x, gr.s1.y, gr.s1.z, gr.s1.w};
    const uint32_t zz[2] = {gr.z.x, gr.z.y};
    // S of activation row 4 g + kq: add the four K blocks' shares, then fetch from a lane that
    // carries that row in its A operand (lane 4 kq of this lane's block of 16)
    float S[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      float v = xsum[g];
      v += __shfl_xor(v, 16, 64);
      v += __shfl_xor(v, 32, 64);
      S[g] = row_lane(v, row_lane0 + 4 * d.kq);
      xsum[g] = 0.f;
    }
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int c = 4 * h + r;                  // column of the word
          const int nib = (c >> 1) + 4 * (c & 1);   // its nibble (AWQ interleave)
          const float zf = (float)((zz[b] >> (4 * nib)) & 0xFu);  // AWQ zero points are used as stored
          const half2_t pr = as_half2(su[(8 * b + c) >> 1]);
          const float sf = (float)((c & 1) ? pr.y : pr.x);
          const float cz = (r < 2 ? kOffLo : kOffHi) + zf;
#pragma unroll
          for (int g = 0; g < G; ++g) tot[8 * b + c][g] = fmaf(sf, acc[b][h][g][r] - cz * S[g], tot[8 * b + c][g]);
        }
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int h = 0; h < 2; ++h) acc[b][h][g] = zero4;
  };

  auto process_step = [&](int st, const uint2_t (&w)[8]) {
    const int k = d.kw0 + st * 32;
    const bool group_end = (st == nsteps - 1) || ((k + 32) % p.groupsize == 0);
    uint4_t xa[G];
#pragma unroll
    for (int g = 0; g < G; ++g) {
      xa[g] = *(const uint4_t*)(smem + a_off[g] + (size_t)st * 64);
      xsum[g] += sum8<DTYPE>(xa[g]);
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      uint2_t a[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const uint32_t pair = (r >> 1) == 0 ? xa[g].x : ((r >> 1) == 1 ? xa[g].y : ((r >> 1) == 2 ? xa[g].z : xa[g].w));
        const uint32_t xx = __builtin_amdgcn_perm(pair, pair, (r & 1) ? 0x03020302u : 0x01000100u);
        a[g] = uint2_t{xx & amask0[g], xx & amask1[g]};
      }
      const uint4_t u0 = lean_unpack<DTYPE>(w[r].x, kc);
      const uint4_t u1 = lean_unpack<DTYPE>(w[r].y, kc);
#pragma unroll
      for (int g = 0; g < G; ++g) {
        acc[0][0][g] = diag_mfma<DTYPE>(a[g], uint2_t{u0.x, u0.y}, acc[0][0][g]);
        acc[0][1][g] = diag_mfma<DTYPE>(a[g], uint2_t{u0.z, u0.w}, acc[0][1][g]);
        acc[1][0][g] = diag_mfma<DTYPE>(a[g], uint2_t{u1.x, u1.y}, acc[1][0][g]);
        acc[1][1][g] = diag_mfma<DTYPE>(a[g], uint2_t{u1.z, u1.w}, acc[1][1][g]);
      }
    }
    if (group_end) {
      flush(gpar);
      if (st + 1 < nsteps) gpar = load_group(min((k + 32) / p.groupsize, p.num_groups - 1));
    }
  };

  int s0 = 0;
  for (; s0 + PF < nsteps; s0 += PF) {
#pragma unroll
    for (int b = 0; b < PF; ++b) {
      process_step(s0 + b, wq[b]);
      load_step(s0 + PF + b, wq[b]);
    }
  }
#pragma unroll
  for (int b = 0; b < PF; ++b) process_step(s0 + b, wq[b]);

  gemv_finish<DTYPE, 16, G, false, true>(gp, d, tot, col0, smem);
}

}  // namespace q4
