// Prefill kernel for the GPTQ layout with contiguous groups: the 128 x 384 tile.
//
// gemm_gptq_kernel covers the output with 128 x 256 tiles, two workgroups of four waves per CU.
// A grid of 257 .. 511 such tiles (4096 x 6144 at M = 2048: 384) leaves half of the CUs with
// one workgroup: one wave per SIMD, nothing to run under that wave's fragment reads and
// unpacking, and the launch lasts as long as a full second round.  This kernel gives every CU
// one workgroup of eight waves instead (two per SIMD) with a tile half as wide again: 128 rows
// x 384 columns, 256 tiles where the other kernel has 384.
//   * Eight waves side by side along N, 48 columns each: three 16-column fragments of
//     v_mfma_f32_16x16x32 (lane (c, kb) supplies the K values 8 kb .. 8 kb + 7 of column c, which
//     is one packed GPTQ word).  A lane owns the three adjacent columns 3 c .. 3 c + 2 of its
//     wave, so the words of a 32-row step come with one 96-bit load; accumulators: 8 row
//     fragments x 3 x 4 = 96 registers.
//   * Weights never touch LDS; they are unpacked in registers to the reference's fp16 value
//     round(s * (q - z)) (dequant_word), two K tiles ahead of their use.
//   * The activation tile (128 rows x 64 K) goes through LDS, double buffered, rows of eight
//     16-byte units in the K order of the nibble splice, unit u of row m at position
//     u ^ ((m >> 1) & 7) (conflict-free 128-bit fragment reads, see q4_gemm_awq_direct.cuh); one
//     barrier per K tile.
// Quantisation groups are multiples of 64 rows (one group per K tile); K is not split.
#pragma once

#include "q4_gemm_awq_direct.cuh"

namespace q4 {

constexpr int kWideBM = 128;
constexpr int kWideBN = 384;

template <int DTYPE>
__global__ __launch_bounds__(512, 1) void gemm_gptq_wide_kernel(GemmParams gp) {
  constexpr int BM = kWideBM;
  constexpr int MT = BM / 16;                    // MFMA row fragments per wave
  constexpr int NF = 3;                          // column fragments (and adjacent columns per lane)
  constexpr int A_LOADS = BM * (kBK / 8) / 512;  // 16-byte activation loads per thread per tile
  constexpr int A_TILE_BYTES = BM * kDirectRowBytes;
  constexpr int FR = kDirectSteps * MT;          // A fragments per K tile
  extern __shared__ __align__(16) unsigned char smem[];  // two activation tiles
  const Problem& p = gp.p;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15;
  const int kb = lane >> 4;
  const int N = p.N, K = p.K, M = p.M;

  // Tile order: workgroup ids go round-robin over the 8 XCDs; every XCD takes a few column
  // blocks and all their M tiles, so a column block's packed words are fetched into one L2.
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_n = N / kWideBN;
  const int total = tiles_m * tiles_n;
  int tm, tn;
  {
    const int bid = blockIdx.x;
    if (total % 8 == 0) {
      const int lin = (bid & 7) * (total >> 3) + (bid >> 3);
      tm = lin % tiles_m;
      tn = lin / tiles_m;
    } else {
      tm = bid % tiles_m;
      tn = bid / tiles_m;
    }
  }
  const int m0 = tm * BM;
  const int nw = tn * kWideBN + wave * (16 * NF);  // first column of this wave
  const int ncol = nw + NF * c16;                  // first of this lane's three columns

  const SpliceK splice = gemm_splice_consts();
  const int KT = K / kBK;
  const int last_tile = KT - 1;

  // ---- packed words: row 8 kt + 4 s + kb, columns ncol .. ncol + 2, two K tiles ahead
  const buffer_rsrc_t wrsrc = make_rsrc(p.qweight, (uint32_t)(K >> 3) * (uint32_t)N * 4u);  // host: below 4 GB
  const uint32_t w_lane = ((uint32_t)kb * (uint32_t)N + (uint32_t)ncol) * 4u;
  const uint32_t step_bytes = (uint32_t)N * 16u;  // four packed rows per 32-row step
  typedef uint32_t uint3_t __attribute__((ext_vector_type(3)));
  struct BWords { uint32_t v[NF]; };
  BWords bq[2][kDirectSteps];
  auto load_b = [&](int kt, int s, BWords& dst) {
    const uint3_t t = __builtin_bit_cast(
        uint3_t, __builtin_amdgcn_raw_buffer_load_b96(wrsrc, w_lane, uniform_u32((uint32_t)(kt * kDirectSteps + s) * step_bytes), 0));
    dst.v[0] = t.x;
    dst.v[1] = t.y;
    dst.v[2] = t.z;
  };

  // ---- group constants of the lane's three columns, rebuilt for every tile from small loads
  // issued one tile earlier
  const buffer_rsrc_t srsrc = make_rsrc(p.scales, (uint32_t)p.num_groups * (uint32_t)N * 2u);
  const buffer_rsrc_t zrsrc = make_rsrc(p.qzeros, (uint32_t)p.num_groups * (uint32_t)(N >> 3) * 4u);
  ColConsts cc[NF];
  uint32_t sraw[NF], zraw[NF];
  auto load_group_raw = [&](int kt) {
    int gi = (kt * kBK) / p.groupsize;
    gi = min(gi, p.num_groups - 1);
    const uint32_t srow = uniform_u32((uint32_t)gi * (uint32_t)N * 2u), zrow = uniform_u32((uint32_t)gi * (uint32_t)(N >> 3) * 4u);
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      sraw[f] = __builtin_amdgcn_raw_buffer_load_b16(srsrc, (uint32_t)(ncol + f) * 2u, srow, 0);
      zraw[f] = __builtin_amdgcn_raw_buffer_load_b32(zrsrc, (uint32_t)((ncol + f) >> 3) * 4u, zrow, 0);
    }
  };
  auto make_group = [&]() {
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const uint32_t z = (gptq_zero_plus_one(zraw[f]) >> (((ncol + f) & 7) * 4)) & 0xFu;
      cc[f] = make_col_consts(z, __builtin_bit_cast(half_t, (uint16_t)sraw[f]));
    }
  };

  // ---- activation tile: global -> registers -> LDS
  const buffer_rsrc_t xrsrc = make_rsrc(p.x, (uint32_t)M * (uint32_t)K * 2u);  // host: below 4 GB
  uint4_t areg[A_LOADS];
  uint32_t a_off[A_LOADS];
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    const int u = tid + 512 * i;
    const int m = u >> 3, ku = u & 7;
    const int row = min(m0 + m, M - 1);  // rows past M re-read the last row; never stored
    a_off[i] = ((uint32_t)row * (uint32_t)K + (uint32_t)ku * 8u) * 2u;
  }
  auto load_a = [&](int kt) {
    const uint32_t tile_off = uniform_u32((uint32_t)kt * (kBK * 2));
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      areg[i] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, a_off[i], tile_off, 0));
  };
  auto store_a = [&](int buf) {
    unsigned char* base = smem + buf * A_TILE_BYTES;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + 512 * i;
      const int m = u >> 3, ku = u & 7;
      const uint4_t v = areg[i];
      uint4_t o;  // K order [0,4,1,5,2,6,3,7] of the splice
      o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
      o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
      o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
      o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
      *(uint4_t*)(base + m * kDirectRowBytes + ((ku ^ ((m >> 1) & 7)) * 16)) = o;
    }
  };

  float4_t acc[MT][NF];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};

  // A fragment g of a tile (g = s * MT + mt): rows 16 mt + c16, K units 4 s + kb (swizzled)
  const int a_swz = (c16 >> 1) & 7;
  const int a_lane_off[kDirectSteps] = {c16 * kDirectRowBytes + ((kb ^ a_swz) * 16), c16 * kDirectRowBytes + (((4 + kb) ^ a_swz) * 16)};
  uint4_t afrag[4];  // rolling window: fragment g sits in slot g % 4, two are read ahead
  auto read_a = [&](int buf, int g) {
    const int s = g / MT, mt = g % MT;
    return *(const uint4_t*)(smem + buf * A_TILE_BYTES + a_lane_off[s] + mt * 16 * kDirectRowBytes);
  };
  uint4_t bfrag[NF];  // the current step's fragments (the second wave of the SIMD covers the unpacking)

  // ---- prologue
  load_a(0);
#pragma unroll
  for (int s = 0; s < kDirectSteps; ++s) load_b(0, s, bq[0][s]);
#pragma unroll
  for (int s = 0; s < kDirectSteps; ++s) load_b(min(1, last_tile), s, bq[1][s]);
  load_group_raw(0);
  store_a(0);
  load_a(min(1, last_tile));
  __syncthreads();
  afrag[0] = read_a(0, 0);
  afrag[1] = read_a(0, 1);

  // The pieces of a K tile.  A step = unpack (vector ALU: three words to 24 halves, then the
  // refill of the freed registers two tiles on) + 24 MFMAs with the A fragments read two ahead.
  // Tile indices past the end are clamped (fetched again, ignored): no branches.
  auto unpack = [&](auto par_c, auto s_c, int kt_refill) {
    constexpr int par = decltype(par_c)::value, s = decltype(s_c)::value;
#pragma unroll
    for (int f = 0; f < NF; ++f) bfrag[f] = dequant_word<DTYPE>(bq[par][s].v[f], cc[f], splice);
    __builtin_amdgcn_sched_barrier(0);  // the unpacking stays in front of the MFMAs that follow
    load_b(kt_refill, s, bq[par][s]);
  };
  // tail_barrier: the last two reads of step 1 cross into the next tile's buffer behind the
  // tile's barrier; otherwise step 1 ends without them (the caller reads them after its barrier)
  auto mfma_step = [&](auto cur_c, auto s_c, auto tail_c) {
    constexpr int cur = decltype(cur_c)::value, s = decltype(s_c)::value;
    constexpr bool tail_barrier = decltype(tail_c)::value;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int g = s * MT + mt;
      const int gn = g + 2;
      if (gn < FR) {
        afrag[gn & 3] = read_a(cur, gn);
      } else if constexpr (tail_barrier) {
        // One barrier per tile: every wave has issued its last reads of this tile's buffer
        // and written its share of the next tile into the other one.
        if (gn == FR) __syncthreads();
        afrag[gn & 3] = read_a(cur ^ 1, gn - FR);
      }
#pragma unroll
      for (int f = 0; f < NF; ++f) acc[mt][f] = mfma16<DTYPE>(afrag[g & 3], bfrag[f], acc[mt][f]);
      // per row fragment: its LDS read, three MFMAs, a share of the step's global loads
      __builtin_amdgcn_sched_group_barrier(0x080, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 3, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
  };
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  // Odd and even waves walk a tile in opposite phase.  The tile barrier keeps the eight waves in
  // step: left alone they all unpack together (vector ALU, the activation tile's LDS writes) and
  // all multiply together (every MFMA group behind a 1 KB fragment read: 85 bytes per clock of
  // the LDS's 128 when all four SIMDs multiply).  Even waves run unpack 0, MFMAs 0, unpack 1,
  // MFMAs 1; odd waves run MFMAs 0, unpack 1, MFMAs 1, unpack 0 of the next tile, and both reach
  // the tile's barrier at the same time.  Measured on 4096 x 6144, same box: M = 1536 86.1 ->
  // 81.4 us, 2000 105.6 -> 102.8, 2048 106.4 -> 105.7; bf16 93.0 -> 87.8, 99.1 -> 95.9, 100.1 ->
  // 97.2.  Splitting the two waves of one SIMD instead (by hardware SIMD id, or w and w + 4)
  // gained nothing.  (Unpacking a step ahead inside one wave, spread between the MFMAs of the
  // step before, measured slower: 110 against 106 us at M = 2048.)
  auto tile_early = [&](int kt, auto cur_c) {
    constexpr int cur = decltype(cur_c)::value;
    using Cur = std::integral_constant<int, cur>;
    const int kt1 = min(kt + 1, last_tile), kt2 = min(kt + 2, last_tile);
    make_group();
    load_group_raw(kt1);
    unpack(Cur{}, I0{}, kt2);
    mfma_step(Cur{}, I0{}, std::true_type{});
    unpack(Cur{}, I1{}, kt2);
    store_a(cur ^ 1);
    load_a(kt2);
    mfma_step(Cur{}, I1{}, std::true_type{});
  };
  auto tile_late = [&](int kt, auto cur_c) {
    constexpr int cur = decltype(cur_c)::value;
    using Cur = std::integral_constant<int, cur>;
    using Nxt = std::integral_constant<int, cur ^ 1>;
    const int kt2 = min(kt + 2, last_tile), kt3 = min(kt + 3, last_tile);
    mfma_step(Cur{}, I0{}, std::true_type{});
    unpack(Cur{}, I1{}, kt2);
    store_a(cur ^ 1);
    load_a(kt2);
    mfma_step(Cur{}, I1{}, std::false_type{});
    make_group();  // the next tile's group (its raw values were asked for a tile ago)
    load_group_raw(kt2);
    unpack(Nxt{}, I0{}, kt3);
    __syncthreads();
    afrag[0] = read_a(cur ^ 1, 0);
    afrag[1] = read_a(cur ^ 1, 1);
  };
  if ((wave & 1) == 0) {
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
      tile_early(kt, I0{});
      tile_early(kt + 1, I1{});
    }
    if (kt < KT) tile_early(kt, I0{});
  } else {
    make_group();
    load_group_raw(min(1, last_tile));
    unpack(I0{}, I0{}, min(2, last_tile));
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
      tile_late(kt, I0{});
      tile_late(kt + 1, I1{});
    }
    if (kt < KT) tile_late(kt, I0{});
  }

  // ---- epilogue.  C layout of the 16x16 MFMA: register r of lane (c16, kb) is row 4 kb + r,
  // column c16 of the fragment, i.e. column ncol + f of the output.  Lanes 2t and 2t + 1 own six
  // adjacent columns, 12 bytes from a 4-byte boundary: the even lane writes columns 0,1 and
  // (with the odd lane's first sum) 2,3; the odd lane writes 4,5.
  const int h = c16 & 1;
  uint16_t* y = (uint16_t*)p.y;
  const bool has_bias = p.bias != nullptr;
  float bias_f[4] = {0.f, 0.f, 0.f, 0.f};
  if (has_bias) {
#pragma unroll
    for (int t = 0; t < 4; ++t) bias_f[t] = load_act<DTYPE>(p.bias, min(ncol + t, N - 1));
  }
  // the sum is rounded to the activation dtype first and the bias added in that dtype
  auto finish = [&](float v, float b) -> uint32_t {
    uint16_t o = store_act<DTYPE>(v);
    if (has_bias) {
      float ob;
      if constexpr (DTYPE == Q4_DTYPE_F16) ob = (float)__builtin_bit_cast(half_t, o);
      else ob = bf16_bits_to_f32(o);
      o = store_act<DTYPE>(ob + b);
    }
    return o;
  };
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float v0 = acc[mt][0][r], v1 = acc[mt][1][r], v2 = acc[mt][2][r];
      const float got = swap_neighbour(v0);  // even lane: first sum of the odd lane (column ncol + 3)
      const int m = m0 + mt * 16 + 4 * kb + r;
      if (m < M) {
        uint16_t* row = y + (size_t)m * N + ncol;
        if (h == 0) {
          *(uint32_t*)row = finish(v0, bias_f[0]) | (finish(v1, bias_f[1]) << 16);
          *(uint32_t*)(row + 2) = finish(v2, bias_f[2]) | (finish(got, bias_f[3]) << 16);
        } else {
          *(uint32_t*)(row + 1) = finish(v1, bias_f[1]) | (finish(v2, bias_f[2]) << 16);
        }
      }
    }
  }
}

}  // namespace q4
