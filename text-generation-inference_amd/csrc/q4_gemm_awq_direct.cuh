// Prefill kernel for the AWQ layout that feeds the packed words to the MFMA from registers
// (server/text_generation_server/layers/awq/quantize/cuda.py:43-49 is the call it serves; the
// checkpoint tensors are read as stored).
//
// An AWQ word holds one K row of eight columns; an MFMA B operand wants eight K values of one
// column per lane.  With v_mfma_f32_16x16x32 lane (c = lane % 16, kb = lane / 16) supplies the
// K values 8 kb .. 8 kb + 7 of column c of a 32 x 16 fragment.  Here a wave owns eight words
// (64 columns); lane c works on word c / 2 and on the four nibble positions 4 (c % 2) .. + 3 of
// it, which hold the logical columns 8 (c / 2) + (c % 2) + {0, 2, 4, 6}
// (layers/awq/conversion_utils.py:5).  It loads that word for each of its eight K rows; one byte
// permute puts the same byte of two rows' words into the two halves of a register, and two
// v_and_or_b32 splice its two nibbles into 1024.0 (low nibble: 1024 + q) and 64.0 (high nibble,
// four bits up, where the mantissa step is 1/16: 64 + q).  Two words thus give one register (two
// consecutive K values) of each of the lane's four B fragments for 2 + 4 operations, and
// (q - z) * s costs one packed add and one packed multiply per register as in the GPTQ kernel:
// the weight is the reference's fp16 value round(s * (q - z)), bit for bit.  Nothing goes through
// LDS but the activation tile, and no word is unpacked twice in a workgroup beyond the two lanes
// that share it (each takes half of its nibbles).
//
// Workgroup: 4 waves side by side along N (BM x 256 tile, BM = 32, 64 or 96), or 8 waves in two
// K groups as in gemm_gptq_kernel.  Fragment f of a lane is column 8 (c / 2) + 2 f + (c % 2) of
// the wave's 64; at the end neighbouring lanes swap two of their four sums so that each owns
// four adjacent columns and writes them with one store.
#pragma once

#include "q4_gemm_kernels.cuh"

namespace q4 {

constexpr int kDirectSteps = kBK / 32;  // MFMA K steps (32 rows) per K tile
// Activation tile in LDS: rows of eight 16-byte units (64 K values), unit u of row m stored at
// position u ^ ((m >> 1) & 7).  A 128-bit LDS read is served sixteen lanes at a time -- lanes
// 0-7 with 24-31, 8-15 with 16-23, and the same in the upper half of the wave (measured: any
// two of those lanes on the same four banks cost a pass) -- so the 16 rows x 2 units such a
// pass touches must fall on 16 different units modulo 16: rows of one parity get the swizzle's
// eight different positions, the other parity sits 128 bytes further on.  The stores (eight
// lanes per row, rows m and m + 3 or m + 1 and m + 2 in a pass) are conflict free as well.
constexpr int kDirectRowBytes = (kBK / 8) * 16;

template <int DTYPE>
struct AwqCol;  // constants of one column within one quantisation group
template <>
struct AwqCol<Q4_DTYPE_F16> {
  half2_t cz;  // -(1024 + z) for low-nibble fragments, -(64 + z) for high-nibble ones
  half2_t s2;  // (s, s)
};
template <>
struct AwqCol<Q4_DTYPE_BF16> {
  float sf;  // float(s)
  float cf;  // -(1024 + z) * float(s) or -(64 + z) * float(s): exact
};

struct AwqSpliceK {
  uint32_t mask_lo, mask_hi, magic_lo, magic_hi;
};
__device__ __forceinline__ AwqSpliceK awq_splice_consts() {
  // register operands, so that (w & mask) | magic selects v_and_or_b32 (see gemm_splice_consts)
  AwqSpliceK k{0x000F000Fu, 0x00F000F0u, 0x64006400u, 0x54005400u};
  asm volatile("" : "+s"(k.mask_lo), "+s"(k.mask_hi), "+v"(k.magic_lo), "+v"(k.magic_hi));
  return k;
}

template <int DTYPE, bool HIGH>
__device__ __forceinline__ AwqCol<DTYPE> make_awq_col(uint32_t z, uint32_t s_bits) {
  AwqCol<DTYPE> c;
  const half_t s = __builtin_bit_cast(half_t, (uint16_t)s_bits);
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    const uint32_t h = HIGH ? (0xD400u | (z << 4)) : (0xE400u | z);
    c.cz = as_half2(h | (h << 16));
    c.s2 = half2_t{s, s};
  } else {
    c.sf = (float)s;
    c.cf = -((HIGH ? 64.f : 1024.f) + (float)z) * c.sf;
  }
  return c;
}

// Words of two consecutive K rows -> register (K pair) of the lane's four fragments.
template <int DTYPE>
__device__ __forceinline__ void awq_unpack_pair(uint32_t w0, uint32_t w1, uint32_t sel0, uint32_t sel1,
                                                const AwqCol<DTYPE> (&c)[4], const AwqSpliceK& k, uint32_t (&o)[4]) {
  const uint32_t y0 = __builtin_amdgcn_perm(w1, w0, sel0);  // byte 2h of both rows
  const uint32_t y1 = __builtin_amdgcn_perm(w1, w0, sel1);  // byte 2h + 1
  const uint32_t v[4] = {(y0 & k.mask_lo) | k.magic_lo, (y0 & k.mask_hi) | k.magic_hi, (y1 & k.mask_lo) | k.magic_lo,
                         (y1 & k.mask_hi) | k.magic_hi};
#pragma unroll
  for (int f = 0; f < 4; ++f) {
    if constexpr (DTYPE == Q4_DTYPE_F16) {
      // exact q - z, then the reference's one fp16 rounding
      o[f] = as_u32((as_half2(v[f]) + c[f].cz) * c[f].s2);
    } else {
      // bf16: float(s) * (q - z) exactly in fp32 (one mixed-precision multiply-add from the
      // spliced half), rounded once by the packed convert
      gemm_float2_t t;
      asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(t.x) : "v"(v[f]), "v"(c[f].sf), "v"(c[f].cf));
      asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(t.y) : "v"(v[f]), "v"(c[f].sf), "v"(c[f].cf));
      o[f] = __builtin_bit_cast(uint32_t, __builtin_convertvector(t, gemm_bf16x2_t));
    }
  }
}

template <int DTYPE>
__device__ __forceinline__ float4_t mfma16(const uint4_t a, const uint4_t b, float4_t c) {
  if constexpr (DTYPE == Q4_DTYPE_F16)
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
}

// value of the neighbouring lane (lanes 2t and 2t + 1 swap)
__device__ __forceinline__ float swap_neighbour(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), 0xB1, 0xF, 0xF, true));
}

// BM: rows per workgroup (32, 64, 96).  KG: K groups per workgroup (2: eight waves, the groups
// take the even / odd K tiles with their own activation buffers and add up through LDS).
// Quantisation groups are multiples of 64 rows (one group per K tile).
// 96 rows is the largest tile that compiles without register spills at two waves per SIMD (a
// 128-row tile spills some 25 registers, and every reload waits for the whole prefetch queue:
// it measured 330 against 255 us on 4096 x 14336 at M = 2048).
template <int DTYPE, int BM, int KG = 1>
__global__ __launch_bounds__(256 * KG, (KG == 2 ? 1 : BM == 32 ? 3 : 2)) void gemm_awq_direct_kernel(GemmParams gp) {
  static_assert(BM == 32 || BM == 64 || BM == 96, "row tiles of 32, 64 or 96");
  static_assert(KG == 1 || BM == 96, "two K groups: 96-row tiles");
  constexpr int MT = BM / 16;                    // MFMA row fragments per wave
  constexpr int A_LOADS = BM * (kBK / 8) / 256;  // 16-byte activation loads per thread per tile
  constexpr int A_TILE_BYTES = BM * kDirectRowBytes;
  constexpr int FR = kDirectSteps * MT;          // A fragments per K tile
  extern __shared__ __align__(16) unsigned char smem[];  // two activation tiles per K group
  const Problem& p = gp.p;
  const int tid = threadIdx.x & 255;
  const int grp = KG == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int c16 = lane & 15;
  const int kb = lane >> 4;
  const int word = c16 >> 1;
  const int h = c16 & 1;
  const int N = p.N, K = p.K, M = p.M;
  const int NWORDS = N >> 3;

  // XCD-aware tile order (workgroup ids go round-robin over the 8 XCDs): with more than one
  // round every XCD keeps its own slice of M tiles (the activations stay in its L2) and walks
  // the column blocks; a single round gives every XCD a few column blocks and all their M tiles.
  const int tiles_m = (M + BM - 1) / BM;
  constexpr int BN = 256;
  const int tiles_n = N / BN;
  const int total_tiles = tiles_m * tiles_n;
  const int split = blockIdx.x / total_tiles;
  int tm, tn;
  {
    const int bid = blockIdx.x - split * total_tiles;
    if (tiles_m % 8 == 0 && total_tiles > 256) {
      const int mpx = tiles_m >> 3;
      const int local = bid >> 3;
      tm = (bid & 7) * mpx + local % mpx;
      tn = local / mpx;
    } else if (total_tiles % 8 == 0) {
      const int lin = (bid & 7) * (total_tiles >> 3) + (bid >> 3);
      tm = lin % tiles_m;
      tn = lin / tiles_m;
    } else {
      tm = bid % tiles_m;
      tn = bid / tiles_m;
    }
  }
  const int m0 = tm * BM;
  const int nw = tn * BN + wave * 64;    // first column of this wave
  const int wword = (nw >> 3) + word;    // this lane's packed word within a row

  const AwqSpliceK splice = awq_splice_consts();
  // byte 2h / 2h + 1 of the two words of a row pair, side by side in the halves of a register
  const uint32_t sel0 = h ? 0x0C060C02u : 0x0C040C00u;
  const uint32_t sel1 = h ? 0x0C070C03u : 0x0C050C01u;
  const int hshift = 16 * h;

  const int KT_all = K / kBK;
  const int kt0 = (int)((long)split * KT_all / gp.splits) + grp;
  const int kt_end = (int)((long)(split + 1) * KT_all / gp.splits);
  const int KT = (kt_end - kt0 + KG - 1) / KG;  // tiles of this K group: kt0, kt0 + KG, ...
  auto ktile = [&](int i) { return kt0 + i * KG; };
  const int last_tile = KT - 1;

  // ---- packed words: rows 64 kt + 32 s + 8 kb + r, r = 0..7, one word each.  bq[s] holds step s
  // of the next tile to unpack and is refilled as soon as it has been unpacked: one K tile ahead.
  const buffer_rsrc_t wrsrc = make_rsrc(p.qweight, (uint32_t)K * (uint32_t)NWORDS * 4u);  // host: below 2 GB
  const uint32_t row_bytes = (uint32_t)NWORDS * 4u;
  const uint32_t w_lane = (uint32_t)(kb * 8) * row_bytes + (uint32_t)wword * 4u;
  struct BWords { uint32_t v[8]; };
  BWords bq[kDirectSteps];
  auto load_b = [&](int kt, int s, BWords& dst) {
    const uint32_t step_off = (uint32_t)(ktile(kt) * kBK + s * 32) * row_bytes;
#pragma unroll
    for (int r = 0; r < 8; ++r)
      dst.v[r] = __builtin_amdgcn_raw_buffer_load_b32(wrsrc, w_lane, uniform_u32(step_off + (uint32_t)r * row_bytes), 0);
  };

  // ---- group constants of the lane's four columns, rebuilt for every tile from two small loads
  // issued one tile earlier
  AwqCol<DTYPE> cc[4];
  uint4_t sraw;
  uint32_t zraw;
  auto load_group_raw = [&](int kt) {
    int gi = (ktile(kt) * kBK) / p.groupsize;
    gi = min(gi, p.num_groups - 1);
    sraw = *(const uint4_t*)(p.scales + (size_t)gi * N + nw + 8 * word);
    zraw = p.qzeros[(size_t)gi * NWORDS + wword];
  };
  auto make_group = [&]() {
    // column 2 f + h of the word: nibble position 4 h + f of the zero word, half h of scale pair f
    const uint32_t z4 = zraw >> hshift;
    cc[0] = make_awq_col<DTYPE, false>(z4 & 0xFu, (sraw.x >> hshift) & 0xFFFFu);
    cc[1] = make_awq_col<DTYPE, true>((z4 >> 4) & 0xFu, (sraw.y >> hshift) & 0xFFFFu);
    cc[2] = make_awq_col<DTYPE, false>((z4 >> 8) & 0xFu, (sraw.z >> hshift) & 0xFFFFu);
    cc[3] = make_awq_col<DTYPE, true>((z4 >> 12) & 0xFu, (sraw.w >> hshift) & 0xFFFFu);
  };

  // ---- activation tile: global -> registers -> LDS (swizzled rows of 8 16-byte units); the
  // registers hold the tile after next from one tile's second step to the next one's
  const buffer_rsrc_t xrsrc = make_rsrc(p.x, (uint32_t)M * (uint32_t)K * 2u);  // host: below 2 GB
  uint4_t areg[A_LOADS];
  uint32_t a_off[A_LOADS];  // byte offset of the thread's units within x
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    const int u = tid + 256 * i;
    const int m = u >> 3, ku = u & 7;
    const int row = min(m0 + m, M - 1);  // rows past M re-read the last row; never stored
    a_off[i] = ((uint32_t)row * (uint32_t)K + (uint32_t)ku * 8u) * 2u;
  }
  auto load_a = [&](int kt) {
    const uint32_t tile_off = uniform_u32((uint32_t)ktile(kt) * (kBK * 2));
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      areg[i] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, a_off[i], tile_off, 0));
  };
  auto store_a = [&](int buf) {
    unsigned char* base = smem + (grp * 2 + buf) * A_TILE_BYTES;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + 256 * i;
      const int m = u >> 3, ku = u & 7;
      *(uint4_t*)(base + m * kDirectRowBytes + ((ku ^ ((m >> 1) & 7)) * 16)) = areg[i];
    }
  };

  float4_t acc[MT][4];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int f = 0; f < 4; ++f) acc[mt][f] = float4_t{0.f, 0.f, 0.f, 0.f};

  // A fragment g of a tile (g = s * MT + mt): rows 16 mt + c16, K units 4 s + kb (swizzled)
  const int a_swz = (c16 >> 1) & 7;
  const int a_lane_off[kDirectSteps] = {c16 * kDirectRowBytes + ((kb ^ a_swz) * 16), c16 * kDirectRowBytes + (((4 + kb) ^ a_swz) * 16)};
  uint4_t afrag[4];  // rolling window: fragment g sits in slot g % 4, two are read ahead
  auto read_a = [&](int buf, int g) {
    const int s = g / MT, mt = g % MT;
    return *(const uint4_t*)(smem + (grp * 2 + buf) * A_TILE_BYTES + a_lane_off[s] + mt * 16 * kDirectRowBytes);
  };
  uint4_t bfrag[4];  // the current step's four fragments (the second wave of the SIMD covers the unpacking)
  auto unpack_step = [&](const BWords& w) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      uint32_t o[4];
      awq_unpack_pair<DTYPE>(w.v[2 * i], w.v[2 * i + 1], sel0, sel1, cc, splice, o);
#pragma unroll
      for (int f = 0; f < 4; ++f) bfrag[f][i] = o[f];
    }
  };

  // ---- prologue
  load_a(0);
  load_b(0, 0, bq[0]);
  load_b(0, 1, bq[1]);
  load_group_raw(0);
  store_a(0);
  load_a(min(1, last_tile));
  __syncthreads();
  afrag[0] = read_a(0, 0);
  afrag[1] = read_a(0, 1);

  // One K tile.  A step unpacks its words, asks for the same step of the next tile into the
  // freed registers and runs its MFMAs with the A fragments read two ahead; the second step
  // moves tile kt + 1 from registers to the other LDS buffer and asks for tile kt + 2.  Tile
  // indices past the end are clamped (fetched again, ignored): no branches.
  auto tile_step = [&](int kt, auto cur_c) {
    constexpr int cur = decltype(cur_c)::value;
    const int kt1 = min(kt + 1, last_tile);
    make_group();
    load_group_raw(kt1);
#pragma unroll
    for (int s = 0; s < kDirectSteps; ++s) {
      unpack_step(bq[s]);
      __builtin_amdgcn_sched_barrier(0);  // the unpacking stays in front of the step's MFMAs
      load_b(kt1, s, bq[s]);
      if (s == 1) {
        store_a(cur ^ 1);
        load_a(min(kt + 2, last_tile));
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int g = s * MT + mt;
        const int gn = g + 2;
        if (gn < FR) {
          afrag[gn & 3] = read_a(cur, gn);
        } else {
          // One barrier per tile: every wave has issued its last reads of this tile's buffer
          // and written its share of the next tile into the other one.
          if (gn == FR) __syncthreads();
          afrag[gn & 3] = read_a(cur ^ 1, gn - FR);
        }
#pragma unroll
        for (int f = 0; f < 4; ++f) acc[mt][f] = mfma16<DTYPE>(afrag[g & 3], bfrag[f], acc[mt][f]);
        // per row fragment: its LDS traffic, four MFMAs, a few of the step's global loads
        __builtin_amdgcn_sched_group_barrier(0x080, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, 4, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 2, 0);
      }
    }
  };
  {
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    int kt = 0;
    for (; kt + 1 < KT; kt += 2) {
      tile_step(kt, I0{});
      tile_step(kt + 1, I1{});
    }
    if (kt < KT) tile_step(kt, I0{});
  }

  if constexpr (KG == 2) {
    __syncthreads();  // the activation buffers are dead
    float* xch = (float*)smem;
    if (grp == 1) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < 4; ++f)
#pragma unroll
          for (int r = 0; r < 4; ++r) xch[((mt * 4 + f) * 4 + r) * 256 + tid] = acc[mt][f][r];
    }
    __syncthreads();
    if (grp == 1) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int f = 0; f < 4; ++f)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[mt][f][r] += xch[((mt * 4 + f) * 4 + r) * 256 + tid];
  }

  // ---- epilogue.  C layout of the 16x16 MFMA: register r of lane (c16, kb) is row 4 kb + r,
  // column c16 of the fragment, i.e. logical column 8 word + 2 f + h.  Lanes 2t (h = 0: columns
  // 0,2,4,6 of the word) and 2t + 1 (1,3,5,7) swap two sums each: the even lane ends up with
  // columns 0..3, the odd one with 4..7.
  const int ncol = nw + 8 * word + 4 * h;
  float* part = gp.splits > 1 ? gp.partials + (size_t)split * gp.partial_rows * N : nullptr;
  uint16_t* y = (uint16_t*)p.y;
  float bias_f[4] = {0.f, 0.f, 0.f, 0.f};
  const bool has_bias = p.bias != nullptr && gp.splits == 1;
  if (has_bias) {
#pragma unroll
    for (int t = 0; t < 4; ++t) bias_f[t] = load_act<DTYPE>(p.bias, ncol + t);
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
      const float v0 = acc[mt][0][r], v1 = acc[mt][1][r], v2 = acc[mt][2][r], v3 = acc[mt][3][r];
      const float got0 = swap_neighbour(h ? v0 : v2);
      const float got1 = swap_neighbour(h ? v1 : v3);
      const float o0 = h ? got0 : v0, o1 = h ? v2 : got0, o2 = h ? got1 : v1, o3 = h ? v3 : got1;
      const int m = m0 + mt * 16 + 4 * kb + r;
      if (m < M) {
        if (part != nullptr) {
          *(float4_t*)(part + (size_t)m * N + ncol) = float4_t{o0, o1, o2, o3};
        } else {
          uint2_t o;
          o.x = finish(o0, bias_f[0]) | (finish(o1, bias_f[1]) << 16);
          o.y = finish(o2, bias_f[2]) | (finish(o3, bias_f[3]) << 16);
          *(uint2_t*)(y + (size_t)m * N + ncol) = o;
        }
      }
    }
  }
}

}  // namespace q4
