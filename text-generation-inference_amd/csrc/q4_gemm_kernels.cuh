// Prefill kernels (device code shared by the translation units that instantiate them).
//
// Prefill path: y[M, N] = x @ dequant(W) for large M on the MFMA units (gfx950).
//
// MFMA-bound: 2*M*N*K flops against 0.5 B/weight of HBM traffic.  Tiling (wave64):
//   * a workgroup of 4 waves owns a BM x 256 output tile; wave w owns columns
//     n0 + 64 w .. + 63 for all BM rows (4 waves side by side along N);
//   * the B operand never touches LDS: a packed GPTQ word holds 8 consecutive K values of
//     one column, which is exactly what lane (column j, K block kq) of a
//     v_mfma_f32_32x32x16 supplies.  Each lane loads two adjacent words (columns
//     nw + 2j, nw + 2j + 1) of packed row K/8 + kq with one 64-bit load (256 contiguous
//     bytes per half-wave), unpacks them in registers to the reference's fp16 weight
//     round_once(s * (q - z)) -- bit-identical to the dense dequantized matrix -- and feeds
//     BM/32 MFMAs with each fragment.  Because the waves split N, no weight is unpacked
//     twice inside a workgroup;
//   * the A operand (activations) is staged through LDS, double buffered, in 16-byte
//     units [row][K block] whose 8 values are stored in the order [0,4,1,5,2,6,3,7] that
//     the nibble splice produces (see q4_common.cuh), so weights are never repacked;
//     the row stride is padded to 9 units, which makes the 128-bit fragment reads
//     conflict free;
//   * packed weights are prefetched two K tiles (128 rows) ahead in registers, activations
//     one tile ahead; fp32 accumulators live in VGPRs (BM = 128: 128 of them, two
//     workgroups per CU so one wave's unpacking overlaps the other's MFMAs).
#pragma once

#include <type_traits>

#include "q4_common.cuh"

namespace q4 {

constexpr int kBK = 64;            // K rows per tile
constexpr int kKSteps = kBK / 16;  // MFMA K steps per tile
constexpr int kAUnitsPerRow = kBK / 8 + 1;  // 16-byte units per LDS row, padded

struct GemmParams {
  Problem p;
  // Split-K for grids that do not fill the chip: `splits` workgroups share an output tile,
  // each takes a contiguous range of K tiles and writes its fp32 partial tile to
  // partials[split][M][N]; gemm_reduce_kernel adds them in split order.  splits == 1:
  // the output is written directly.
  float* __restrict__ partials;
  int splits;
  int partial_rows;  // rows of one split's slice of `partials` (M; grouped launches: all pairs)
  MoeView moe;  // grouped launches only (MOE kernels): blockIdx.y is the expert
};

typedef float float2_t __attribute__((ext_vector_type(2)));
typedef float gemm_float2_t __attribute__((ext_vector_type(2)));
typedef __bf16 gemm_bf16x2_t __attribute__((ext_vector_type(2)));

// Buffer loads: the base sits in a scalar resource descriptor, the lane's part of the address is
// a 32-bit byte offset in one vector register that never changes, and what moves from load to
// load is a scalar offset: no 64-bit vector address arithmetic and no address registers.
typedef __amdgpu_buffer_rsrc_t buffer_rsrc_t;
__device__ __forceinline__ buffer_rsrc_t make_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint32_t uniform_u32(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

struct SpliceK {
  uint32_t mask_lo, mask_hi, magic;
};
__device__ __forceinline__ SpliceK gemm_splice_consts() {
  // Hidden from constant folding so that (w & mask) | magic selects v_and_or_b32 (a
  // three-operand VALU op cannot carry literals).  The asm is empty on purpose.
  SpliceK k{0x000F000Fu, 0x00F000F0u, 0x64006400u};
  asm volatile("" : "+s"(k.mask_lo), "+s"(k.mask_hi), "+v"(k.magic));
  return k;
}

// Per-column constants of one quantisation group.
struct ColConsts {
  half2_t czlo, czhi;  // -(1024 + z), -(64 + z), both halves equal
  half2_t s2;          // (s, s)
  // bf16 path: float(s), float(s) / 16, -(1024 + z) * float(s), -(64 + z) * float(s) (all exact)
  float sf, sf16, clo, chi;
};

__device__ __forceinline__ ColConsts make_col_consts(uint32_t z, half_t s) {
  ColConsts c;
  c.czlo = as_half2(0xE400E400u | z | (z << 16));
  c.czhi = as_half2(0xD400D400u | (z << 4) | (z << 20));
  c.s2 = half2_t{s, s};
  c.sf = (float)s;
  c.sf16 = c.sf * 0.0625f;
  c.clo = -(1024.f + (float)z) * c.sf;
  c.chi = -(64.f + (float)z) * c.sf;
  return c;
}

// One packed word -> MFMA B fragment (8 weights of one column, K order 0,4,1,5,2,6,3,7).
template <int DTYPE>
__device__ __forceinline__ uint4_t dequant_word(uint32_t w, const ColConsts& c, const SpliceK& k) {
  const uint32_t w8 = w >> 8;
  uint4_t out;
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    half2_t d[4];  // exact (q - z)
    d[0] = as_half2((w & k.mask_lo) | k.magic) + c.czlo;
    d[1] = as_half2((w & k.mask_hi) | k.magic) * sixteenth + c.czhi;
    d[2] = as_half2((w8 & k.mask_lo) | k.magic) + c.czlo;
    d[3] = as_half2((w8 & k.mask_hi) | k.magic) * sixteenth + c.czhi;
    // one fp16 multiply per weight: the reference's rounding
    out.x = as_u32(d[0] * c.s2);
    out.y = as_u32(d[1] * c.s2);
    out.z = as_u32(d[2] * c.s2);
    out.w = as_u32(d[3] * c.s2);
  } else {
    // bf16: the exact fp32 value float(s) * (q - z), rounded once to nearest even by the packed
    // convert.  One mixed-precision multiply-add per weight gives it straight from the spliced
    // half: (1024 + q) * s - (1024 + z) * s, or (1024 + 16 q) * s / 16 - (64 + z) * s; both
    // products and both addends are exact in fp32 (the compiler would emit a convert, a
    // subtraction and a multiply instead).
    const uint32_t v[4] = {(w & k.mask_lo) | k.magic, (w & k.mask_hi) | k.magic, (w8 & k.mask_lo) | k.magic,
                           (w8 & k.mask_hi) | k.magic};
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float sc = (i & 1) ? c.sf16 : c.sf, add = (i & 1) ? c.chi : c.clo;
      gemm_float2_t f;
      asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[0,0,0] op_sel_hi:[1,0,0]" : "=v"(f.x) : "v"(v[i]), "v"(sc), "v"(add));
      asm("v_fma_mix_f32 %0, %1, %2, %3 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "=v"(f.y) : "v"(v[i]), "v"(sc), "v"(add));
      o[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, gemm_bf16x2_t));
    }
    out.x = o[0]; out.y = o[1]; out.z = o[2]; out.w = o[3];
  }
  return out;
}

template <int DTYPE>
__device__ __forceinline__ float16_t mfma32(const uint4_t a, const uint4_t b, float16_t c) {
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a),
                                                  __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                   __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  }
}

// BM: rows per workgroup (64, 128 or 256).  GPT: quantisation groups per K tile (1 or 2).
// NW: packed words (columns) per lane and K step: 2 -> 256-column workgroup tile, 1 -> 128.
// MOE: grouped launch, blockIdx.y is the expert; its row count is read from device memory, so
// the grid covers the largest possible count and surplus workgroups leave at once.
// KG: K groups per workgroup (1 or 2).  With 2 the workgroup has eight waves: waves 0-3 take
// the even K tiles of the workgroup's range, waves 4-7 the odd ones, each group with its own
// activation buffers in LDS; the two accumulator sets meet through LDS at the end.  A grid of
// one workgroup per CU then runs two waves per SIMD (one wave's fragment reads and unpacking
// under the other's MFMAs) without any partial tile going through memory.
// FUSE: the weight packs [gate | up] and the output is act(gate) * up, [M, N/2].  A workgroup
// covers 128 gate columns (waves 0, 1) and the 128 up columns that go with them (waves 2, 3):
// the K loop is the plain one, at the end the up waves hand their rounded tile to the gate
// waves through LDS (the activation tiles are dead by then).
template <int DTYPE, int BM, int GPT, int NW, bool MOE = false, int KG = 1, bool FUSE = false>
__global__ __launch_bounds__(256 * KG, (KG == 2 ? 1 : BM == 64 ? 3 : BM == 128 ? (NW == 1 ? (GPT == 1 ? 3 : 1) : 2) : 1)) void gemm_gptq_kernel(GemmParams gp) {
  static_assert(KG == 1 || (KG == 2 && !MOE && BM <= 128), "two K groups: dense launches, at most 128 rows");
  static_assert(!FUSE || (NW == 2 && KG == 1 && !MOE), "gated epilogue: two columns per lane, dense launches, one K group");
  int moe_row0 = 0;
  if constexpr (MOE) {
    moe_row0 = moe_enter(gp.p, gp.moe, blockIdx.y);
    if (gp.p.M <= 0) return;
  }
  constexpr int MT = BM / 32;                      // MFMA row tiles per wave
  constexpr int A_LOADS = BM * (kBK / 8) / 256;    // 16-byte activation loads per thread per tile
  constexpr int A_TILE_BYTES = BM * kAUnitsPerRow * 16;
  extern __shared__ __align__(16) unsigned char smem[];  // two activation tiles
  const Problem& p = gp.p;
  const int tid = threadIdx.x & 255;  // thread of its K group
  const int grp = KG == 1 ? 0 : __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 8));
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int j = lane & 31;
  const int kq = lane >> 5;
  const int N = p.N, K = p.K, M = p.M;

  // XCD-aware tile order.  Workgroup ids are dealt round-robin to the 8 XCDs (id % 8), each
  // with its own L2.  Every XCD is given its own slice of M tiles and walks all column
  // blocks of it: the activation rows of the slice (BM x K, a few MB) stay resident in that
  // XCD's L2 and are re-read from there by every column block, while the packed weights are
  // the streamed operand (each column block is read once per XCD, prefetched ahead).
  // (A grid of a single round, at most one workgroup per CU, measured faster the other way
  // round: each XCD takes a few column blocks and all M tiles of them.)
  const int tiles_m = (M + BM - 1) / BM;
  constexpr int BN = 4 * 32 * NW;
  const int tiles_n = N / BN;
  int tm, tn;
  const int total_tiles = tiles_m * tiles_n;
  if constexpr (MOE) {
    if ((int)blockIdx.x >= total_tiles * gp.splits) return;
  }
  const int split = blockIdx.x / total_tiles;  // workgroups of one split are neighbours in id
  {
    const int bid = blockIdx.x - split * total_tiles;
    const int total = total_tiles;
    if (tiles_m % 8 == 0 && total > 256) {
      const int mpx = tiles_m >> 3;  // M tiles per XCD
      const int xcd = bid & 7;
      const int local = bid >> 3;
      tm = xcd * mpx + local % mpx;
      tn = local / mpx;
    } else if (total % 8 == 0) {
      const int lin = (bid & 7) * (total >> 3) + (bid >> 3);
      tm = lin % tiles_m;
      tn = lin / tiles_m;
    } else {
      tm = bid % tiles_m;
      tn = bid / tiles_m;
    }
  }
  const int m0 = tm * BM;
  const int n0 = tn * BN;
  const int up_off = N >> 1;  // FUSE: first up column
  // first column of this wave
  const int nw = FUSE ? (n0 >> 1) + (wave & 1) * 32 * NW + (wave >> 1) * up_off : n0 + wave * 32 * NW;
  const int ncol = nw + NW * j;  // first of this lane's NW columns

  const SpliceK splice = gemm_splice_consts();
  const int KT_all = K / kBK;
  // this workgroup's K tiles [kt_begin, kt_end); group grp walks kt_begin + grp, + KG, ...
  // (KG == 2: the host makes the count even).  Below, tile indices are positions in the group's
  // own sequence: tile i is K tile kt0 + i * KG.
  const int kt0 = (int)((long)split * KT_all / gp.splits) + grp;
  const int kt_end = (int)((long)(split + 1) * KT_all / gp.splits);
  const int kt_begin = 0;
  const int KT = (kt_end - kt0 + KG - 1) / KG;
  auto ktile = [&](int i) { return kt0 + i * KG; };

  // ---- packed-weight stream: words [K/8 + kq][ncol, ncol+1], two K tiles ahead
  // (buffer loads: scalar descriptor, constant lane offset, scalar step offset; the host keeps
  // the weight and activation byte counts below 4 GB)
  const buffer_rsrc_t wrsrc = make_rsrc(p.qweight, (uint32_t)(K >> 3) * (uint32_t)N * 4u);
  const uint32_t w_lane = ((uint32_t)kq * (uint32_t)N + (uint32_t)ncol) * 4u;
  const uint32_t kstep_bytes = (uint32_t)N * 8u;  // two packed rows per MFMA K step
  struct BWords { uint32_t v[NW]; };
  BWords bq[2][kKSteps];
  auto load_b = [&](int kt, BWords (&dst)[kKSteps]) {
#pragma unroll
    for (int s = 0; s < kKSteps; ++s)
    {
      const uint32_t soff = uniform_u32((uint32_t)(ktile(kt) * kKSteps + s) * kstep_bytes);
      if constexpr (NW == 2) {
        const uint2_t t = __builtin_bit_cast(uint2_t, __builtin_amdgcn_raw_buffer_load_b64(wrsrc, w_lane, soff, 0));
        dst[s].v[0] = t.x; dst[s].v[1] = t.y;
      } else {
        dst[s].v[0] = __builtin_amdgcn_raw_buffer_load_b32(wrsrc, w_lane, soff, 0);
      }
    }
  };

  // ---- group constants for this lane's two columns.  They are rebuilt for every tile
  // from two tiny (cached) loads, which keeps the steady-state loop free of branches.
  ColConsts cc[GPT][NW], cc_next[GPT][NW];
  uint32_t sraw[GPT], zraw[GPT];
  const buffer_rsrc_t srsrc = make_rsrc(p.scales, (uint32_t)p.num_groups * (uint32_t)N * 2u);
  const buffer_rsrc_t zrsrc = make_rsrc(p.qzeros, (uint32_t)p.num_groups * (uint32_t)(N >> 3) * 4u);
  const int zshift = (ncol & 7) * 4;
  auto load_group_raw = [&](int kt) {
#pragma unroll
    for (int g = 0; g < GPT; ++g) {
      int gi = (ktile(kt) * kBK + g * (kBK / GPT)) / p.groupsize;
      gi = min(gi, p.num_groups - 1);
      if constexpr (NW == 2) sraw[g] = __builtin_amdgcn_raw_buffer_load_b32(srsrc, (uint32_t)ncol * 2u, uniform_u32((uint32_t)gi * (uint32_t)N * 2u), 0);
      else sraw[g] = __builtin_amdgcn_raw_buffer_load_b16(srsrc, (uint32_t)ncol * 2u, uniform_u32((uint32_t)gi * (uint32_t)N * 2u), 0);
      zraw[g] = __builtin_amdgcn_raw_buffer_load_b32(zrsrc, (uint32_t)(ncol >> 3) * 4u, uniform_u32((uint32_t)gi * (uint32_t)(N >> 3) * 4u), 0);
    }
  };
  auto make_group = [&](ColConsts (&dst)[GPT][NW]) {
#pragma unroll
    for (int g = 0; g < GPT; ++g) {
      const uint32_t z2 = gptq_zero_plus_one(zraw[g]) >> zshift;
      const half2_t s01 = as_half2(sraw[g]);
      dst[g][0] = make_col_consts(z2 & 0xFu, s01.x);
      if constexpr (NW == 2) dst[g][1] = make_col_consts((z2 >> 4) & 0xFu, s01.y);
    }
  };

  // ---- activation tile: global -> registers -> (permuted) LDS
  // rows of x behind p.x: M, or every token of a grouped launch (its row map points anywhere)
  const buffer_rsrc_t xrsrc = make_rsrc(p.x, 0xFFFFFFFFu);
  // Register staging sets: with two sets (128-row tiles) a tile's loads are issued two
  // tiles before they are written to LDS; the 256-row tile has registers for one set only.
  constexpr int ASETS = BM <= 128 ? 2 : 1;
  uint4_t areg[ASETS][A_LOADS];
  uint32_t a_off[A_LOADS];  // byte offset of the thread's 16-byte units within x (below 4 GB: host)
#pragma unroll
  for (int i = 0; i < A_LOADS; ++i) {
    const int u = tid + 256 * i;
    const int m = u >> 3, kb = u & 7;
    // rows past M re-read the last row: their results are never stored
    int row = min(m0 + m, M - 1);
    if constexpr (MOE) {
      // grouped launch with a row map: x row of each staged row
      if (gp.moe.x_rows != nullptr) row = gp.moe.x_rows[moe_row0 + row];
    }
    a_off[i] = ((uint32_t)row * (uint32_t)K + (uint32_t)kb * 8u) * 2u;
  }
  auto load_a = [&](int kt, auto set_c) {
    constexpr int set = decltype(set_c)::value % ASETS;
    const uint32_t tile_off = uniform_u32((uint32_t)ktile(kt) * (kBK * 2));
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i)
      areg[set][i] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(xrsrc, a_off[i], tile_off, 0));
  };
  auto store_a = [&](int buf, auto set_c) {
    constexpr int set = decltype(set_c)::value % ASETS;
    unsigned char* base = smem + (grp * 2 + buf) * A_TILE_BYTES;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + 256 * i;
      const int m = u >> 3, kb = u & 7;
      const uint4_t v = areg[set][i];
      // K order [0,4,1,5,2,6,3,7] of the splice: one byte permute per register
      uint4_t o;
      o.x = __builtin_amdgcn_perm(v.z, v.x, 0x05040100u);
      o.y = __builtin_amdgcn_perm(v.z, v.x, 0x07060302u);
      o.z = __builtin_amdgcn_perm(v.w, v.y, 0x05040100u);
      o.w = __builtin_amdgcn_perm(v.w, v.y, 0x07060302u);
      *(uint4_t*)(base + (m * kAUnitsPerRow + kb) * 16) = o;
    }
  };

  float16_t acc[MT][NW];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int f = 0; f < NW; ++f)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[mt][f][r] = 0.f;

  const int a_lane_off = (j * kAUnitsPerRow + kq) * 16;
  uint4_t afrag[2][MT];  // A fragments of the current / next MFMA K step
  uint4_t bfrag[2][NW];  // unpacked B fragments of the current / next step
  auto read_a = [&](int buf, int s, uint4_t (&dst)[MT]) {
    const unsigned char* abase = smem + (grp * 2 + buf) * A_TILE_BYTES + a_lane_off;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
      dst[mt] = *(const uint4_t*)(abase + (mt * 32 * kAUnitsPerRow + 2 * s) * 16);
  };
  auto group_of_step = [](int s) { return GPT == 1 ? 0 : (s * 16) / (kBK / GPT); };

  // ---- prologue: tile 0 staged, tile 1 in flight, first fragments ready
  const int last_tile = KT - 1;
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  load_a(kt_begin, I0{});
  load_b(kt_begin, bq[0]);
  load_b(min(kt_begin + 1, last_tile), bq[1]);
  load_group_raw(kt_begin);
  if constexpr (ASETS == 2) load_a(min(kt_begin + 1, last_tile), I1{});
  store_a(0, I0{});
  if constexpr (ASETS == 2) load_a(min(kt_begin + 2, last_tile), I0{});
  else load_a(min(kt_begin + 1, last_tile), I0{});
  make_group(cc);
  __syncthreads();
  read_a(0, 0, afrag[0]);
#pragma unroll
  for (int f = 0; f < NW; ++f) bfrag[0][f] = dequant_word<DTYPE>(bq[0][0].v[f], cc[0][f], splice);

  // One K tile, software pipelined: while the MFMAs of step s run, the VALU unpacks the
  // weights of step s+1 and the LDS returns its A fragments; the global loads of tile
  // kt+2 and the LDS writes of tile kt+1 are spread over the steps.  Tile indices past the
  // end are clamped (the last tile is fetched again and ignored) so the body has no
  // branches and the scheduler sees one region per step.  `cur` selects the LDS buffer and
  // the weight-register set at compile time; the loop is unrolled by two.
  auto tile_step = [&](int kt, auto cur_c) {
    constexpr int cur = decltype(cur_c)::value;
    const int kt1 = min(kt + 1, last_tile);
    const int kt2 = min(kt + 2, last_tile);
#pragma unroll
    for (int s = 0; s < kKSteps; ++s) {
      const int sb = s & 1;
      // (1) LDS reads of the next step's A fragments go first so that they get the early
      // LDS slots of this step.  The last step reads the first fragments of tile kt+1 from
      // the other buffer, which the barrier below (between steps 2 and 3) has published.
      if (s + 1 < kKSteps) read_a(cur, s + 1, afrag[sb ^ 1]);
      else read_a(cur ^ 1, 0, afrag[sb ^ 1]);
      // (2) unpack the next step's weights
      if (s + 1 < kKSteps) {
        const int g = group_of_step(s + 1);
#pragma unroll
        for (int f = 0; f < NW; ++f)
          bfrag[sb ^ 1][f] = dequant_word<DTYPE>(bq[cur][s + 1].v[f], cc[g][f], splice);
      } else {
#pragma unroll
        for (int f = 0; f < NW; ++f)
          bfrag[sb ^ 1][f] = dequant_word<DTYPE>(bq[cur ^ 1][0].v[f], cc_next[0][f], splice);
      }
      // (3) side work of this step
      if (s == 0) {
        // tile kt+1 (staged in register set (kt+1) % ASETS) -> the other LDS buffer
        store_a(cur ^ 1, std::integral_constant<int, cur ^ 1>{});
        load_group_raw(kt1);    // scales / zero points the next tile starts with
      }
      if (s == 1) {
        // refill the set that was just written out: tile kt+3 with two sets, kt+2 with one
        if constexpr (ASETS == 2) load_a(min(kt + 3, last_tile), std::integral_constant<int, cur ^ 1>{});
        else load_a(kt2, I0{});
      }
      if (s == 2) make_group(cc_next);
      // (4) the MFMAs of this step
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int f = 0; f < NW; ++f) acc[mt][f] = mfma32<DTYPE>(afrag[sb][mt], bfrag[sb][f], acc[mt][f]);
      }
      if (s == kKSteps - 1) load_b(kt2, bq[cur]);
      // interleave: after every MFMA a few VALU ops, one LDS op and one global load
#pragma unroll
      for (int i = 0; i < NW * MT; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 7, 0);
        __builtin_amdgcn_sched_group_barrier(0x080, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
      }
      if (s == kKSteps - 2) {
        // One barrier per tile.  Here every wave has finished reading this tile's buffer
        // (the step-3 fragments were read above) and has written its share of the next
        // tile into the other buffer (step 0), so after the barrier the other buffer may
        // be read (step 3) and this one overwritten (step 0 of the next tile).
        __syncthreads();
      }
    }
#pragma unroll
    for (int g = 0; g < GPT; ++g) {
#pragma unroll
      for (int f = 0; f < NW; ++f) cc[g][f] = cc_next[g][f];
    }
  };
  {
    int kt = kt_begin;
    for (; kt + 1 < KT; kt += 2) {
      tile_step(kt, std::integral_constant<int, 0>{});
      tile_step(kt + 1, std::integral_constant<int, 1>{});
    }
    if (kt < KT) tile_step(kt, std::integral_constant<int, 0>{});
  }

  if constexpr (KG == 2) {
    // the odd-tile group hands its sums over through LDS (the activation buffers are dead):
    // accumulator register by register, consecutive threads at consecutive addresses
    __syncthreads();
    float* xch = (float*)smem;
    if (grp == 1) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int f = 0; f < NW; ++f)
#pragma unroll
          for (int r = 0; r < 16; ++r) xch[((mt * NW + f) * 16 + r) * 256 + tid] = acc[mt][f][r];
    }
    __syncthreads();
    if (grp == 1) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int f = 0; f < NW; ++f)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mt][f][r] += xch[((mt * NW + f) * 16 + r) * 256 + tid];
  }

  // ---- epilogue: C layout of the 32x32 MFMA: register r of lane (j, kq) is row
  // 8*(r/4) + 4*kq + r%4, column j.  Fragments 0/1 are adjacent columns -> one 32-bit store.
  if (gp.splits > 1) {
    // fp32 partial tile; bias, rounding and the store to y happen in the reduction kernel
    float* part = gp.partials + ((size_t)split * gp.partial_rows + moe_row0) * N;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + mt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
        if (m < M) {
          if constexpr (NW == 2) *(float2_t*)(part + (size_t)m * N + ncol) = float2_t{acc[mt][0][r], acc[mt][1][r]};
          else part[(size_t)m * N + ncol] = acc[mt][0][r];
        }
      }
    }
    return;
  }
  uint16_t* y = (uint16_t*)p.y;
  float bias_f[NW] = {};
  const bool has_bias = p.bias != nullptr;
  if (has_bias) {
#pragma unroll
    for (int f = 0; f < NW; ++f) bias_f[f] = load_act<DTYPE>(p.bias, ncol + f);
  }
  // The sum is rounded to the activation dtype first and the bias added in that dtype
  // (one more rounding), like `out + bias` on a half tensor.
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
  if constexpr (FUSE) {
    // act(gate) * up on the rounded halves (what the two-kernel route computes).  Every wave
    // leaves its tile in LDS, two halves per word, under (wave, row tile, register, lane); then
    // all threads walk the gate words, each with the up word 2 waves further on.
    constexpr int WORDS = 2 * MT * 16 * 64;  // gate words of the workgroup (as many up words)
    uint32_t* xch = (uint32_t*)smem;
    __syncthreads();  // every wave is done with the activation tiles
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int r = 0; r < 16; ++r)
        xch[((wave * MT + mt) * 16 + r) * 64 + lane] = finish(acc[mt][0][r], bias_f[0]) | (finish(acc[mt][1][r], bias_f[1]) << 16);
    __syncthreads();
    auto product = [&](auto act_c) {
      constexpr int ACT = decltype(act_c)::value;
#pragma unroll 4
      for (int idx = tid; idx < WORDS; idx += 256) {
        const uint32_t g = xch[idx], u = xch[idx + WORDS];
        const int ln = idx & 63, rr = (idx >> 6) & 15, mtt = (idx >> 10) % MT, wv = idx / (1024 * MT);
        const int m = m0 + mtt * 32 + 8 * (rr >> 2) + 4 * (ln >> 5) + (rr & 3);
        const uint32_t lo = act_mul_as<DTYPE, ACT>((uint16_t)(g & 0xFFFFu), (uint16_t)(u & 0xFFFFu));
        const uint32_t hi = act_mul_as<DTYPE, ACT>((uint16_t)(g >> 16), (uint16_t)(u >> 16));
        if (m < M) *(uint32_t*)(y + (size_t)m * up_off + (n0 >> 1) + wv * 64 + 2 * (ln & 31)) = lo | (hi << 16);
      }
    };
    const int act = p.gate_up_act - 1;
    if (act == Q4_ACT_SILU) product(std::integral_constant<int, Q4_ACT_SILU>{});
    else if (act == Q4_ACT_GELU_TANH) product(std::integral_constant<int, Q4_ACT_GELU_TANH>{});
    else product(std::integral_constant<int, Q4_ACT_GELU>{});
    return;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int m = m0 + mt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
      if (m < M) {
        const uint32_t lo = finish(acc[mt][0][r], bias_f[0]);
        if constexpr (NW == 2) {
          const uint32_t hi = finish(acc[mt][1][r], bias_f[1]);
          *(uint32_t*)(y + (size_t)m * N + ncol) = lo | (hi << 16);
        } else {
          y[(size_t)m * N + ncol] = (uint16_t)lo;
        }
      }
    }
  }
}

// y[m][n] = round(sum over splits of partials[s][m][n]) (+ bias), four columns per thread.
template <int DTYPE>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(const float* __restrict__ partials,
                                                          const void* __restrict__ bias, uint16_t* __restrict__ y,
                                                          int M, int N, int splits) {
  const long quads = (long)M * (N >> 2);
  const size_t stride = (size_t)M * N;
  for (long q = (long)blockIdx.x * blockDim.x + threadIdx.x; q < quads; q += (long)gridDim.x * blockDim.x) {
    const size_t e = (size_t)q * 4;
    const int n = (int)(e % (size_t)N);
    // four splits' loads in flight at a time (the partial tiles come from other XCDs' write-backs:
    // a load per loop iteration would pay one memory round trip per split); summed in split order
    float4_t sum = *(const float4_t*)(partials + e);
    int sp = 1;
    for (; sp + 4 <= splits; sp += 4) {
      float4_t v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = *(const float4_t*)(partials + (size_t)(sp + u) * stride + e);
#pragma unroll
      for (int u = 0; u < 4; ++u) { sum.x += v[u].x; sum.y += v[u].y; sum.z += v[u].z; sum.w += v[u].w; }
    }
    for (; sp < splits; ++sp) {
      const float4_t v = *(const float4_t*)(partials + (size_t)sp * stride + e);
      sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
    uint2_t o;
    o.x = (uint32_t)finish_output<DTYPE>(sum.x, bias, n) | ((uint32_t)finish_output<DTYPE>(sum.y, bias, n + 1) << 16);
    o.y = (uint32_t)finish_output<DTYPE>(sum.z, bias, n + 2) | ((uint32_t)finish_output<DTYPE>(sum.w, bias, n + 3) << 16);
    *(uint2_t*)(y + e) = o;
  }
}

}  // namespace q4

