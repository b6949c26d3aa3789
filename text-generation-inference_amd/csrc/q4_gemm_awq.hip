// Prefill path for the layouts whose packed words cannot feed the MFMA directly:
// y[M, N] = x @ dequant(W) for AWQ and for GPTQ with g_idx (act-order), gfx950.
//
// An AWQ word holds 8 interleaved columns of ONE K row; an act-order GPTQ word holds 8 K
// rows that each belong to a different group.  In both cases the weight tile is unpacked
// cooperatively into LDS (the classic dequantize-to-LDS stage) and both MFMA operands are
// read from there:
//   * AWQ workgroup = 4 waves in a 2 x 2 arrangement, tile 128 x 128, K tile 64; each wave owns
//     a 64 x 64 block = 2 x 2 MFMA tiles of v_mfma_f32_32x32x16 (64 accumulator VGPRs),
//     so two workgroups share a CU and cover each other's barriers;
//   * AWQ producer: thread t < 128 owns an 8-row x 1-word patch (8 rows of one K block, 8
//     columns).  One byte permute per row pair and byte puts the same nibble positions of
//     two rows side by side, the mantissa splice turns them into halves, zero points are
//     subtracted exactly and each weight is multiplied once by its fp16 scale (the
//     reference's rounding).  The patch becomes eight 16-byte units (one per column,
//     8 consecutive K values each) written to LDS at [K block][column];
//   * act-order workgroup = 8 waves, 4 x 2, a 32 x 64 block each, same tile.  Producer: wave w
//     owns K block w of the tile, its lanes two adjacent columns each (one 8-byte load for the
//     two packed words).  The groups of the 8 rows (g_idx[k], the same for the whole wave,
//     requested two tiles ahead) index a per-workgroup LDS table of all groups x the tile's
//     128 columns, filled once in the prologue: one LDS read per row fetches the parameters of
//     both columns, and scale and zero point are applied per weight -- no row of qweight is
//     ever moved.  The table holds one 32-bit entry per group and column (fp16 scale | fp16
//     -(1024 + zero)) for up to 184 groups, or an fp16 scale and a zero-point byte for up to
//     245 groups; layers with more groups gather the two values per row from the checkpoint
//     tensors;
//   * LDS layouts: activations [row][K block] with the row stride padded to 9 units,
//     weights [K block][column] with the low column bits XORed with the word index; both
//     give conflict-free 128-bit fragment reads, and the swizzle spreads the AWQ
//     producer's stores (16 words, columns 8 apart) over all banks;
//   * double-buffered LDS, global loads for tile k+2 in flight while tile k is multiplied.
#include "q4_common.cuh"

namespace q4 {

constexpr int kABM = 128;  // rows per workgroup
constexpr int kABN = 128;  // columns per workgroup
constexpr int kABK = 64;   // K rows per tile
constexpr int kAUnits = kABK / 8 + 1;  // padded units per activation row
constexpr size_t kLdsBytesPerWorkgroup = 160 * 1024;  // gfx950: 160 KB of LDS per CU

struct AwqGemmParams {
  // split-K as in the GPTQ GEMM: `splits` workgroups per output tile, fp32 partial tiles in
  // partials[split][M][N], combined by gemm_reduce_kernel
  float* __restrict__ partials;
  int splits;
  int partial_rows;  // rows of one split's slice of `partials` (M; grouped launches: all pairs)
  Problem p;
  MoeView moe;  // grouped launches only (MOE kernels): blockIdx.y is the expert
};

struct AwqSplice {
  uint32_t mask_lo, mask_hi, magic;
};
__device__ __forceinline__ AwqSplice awq_splice_consts() {
  // registers instead of literals so that (w & mask) | magic selects v_and_or_b32
  AwqSplice k{0x000F000Fu, 0x00F000F0u, 0x64006400u};
  asm volatile("" : "+s"(k.mask_lo), "+s"(k.mask_hi), "+v"(k.magic));
  return k;
}

// LDS slot of a weight unit inside its K block: the low three column bits are XORed with the
// column's word index.  The AWQ producer stores one nibble position of 16 words per
// instruction (columns 8 apart: without the swizzle every lane would hit the same banks);
// consumers read 32 consecutive columns, which the swizzle only permutes.
__device__ __forceinline__ int b_slot(int n) { return n ^ ((n >> 3) & 7); }

typedef __bf16 awq_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float awq_float2_t __attribute__((ext_vector_type(2)));

constexpr int kModeAwq = 0;        // AWQ layout
constexpr int kModeActGather = 1;  // GPTQ layout with g_idx, per-row parameters from global memory
constexpr int kModeActWide = 2;    // GPTQ layout with g_idx, LDS table of 32-bit (scale | -(1024 + zero)) entries
constexpr int kModeActNarrow = 3;  // GPTQ layout with g_idx, LDS table of fp16 scales and zero-point bytes
constexpr int kActWideGroupBytes = kABN * 4;
constexpr int kActNarrowGroupBytes = kABN * 3;  // 128 fp16 scales, then 128 zero-point bytes

// MOE: grouped launch, blockIdx.y is the expert; its row count is read from device memory, so
// the grid covers the largest possible count and surplus workgroups leave at once.
template <int DTYPE, int MODE, bool MOE = false, int BM = kABM>
__global__ __launch_bounds__(MODE == kModeAwq ? 256 : 512, 2) void gemm_awq_kernel(AwqGemmParams gp) {
  constexpr bool ACT = MODE != kModeAwq;
  static_assert(BM == kABM || (BM == 2 * kABM && ACT), "256-row tiles: act-order only");
  // AWQ: 4 waves, 2 x 2, a 64 x 64 block each.  Act-order: 8 waves, 4 x 2, a 32 x 64 block each: the
  // parameter table leaves room for one workgroup per CU, and a single wave per SIMD cannot hide
  // its own LDS and unpack latencies behind its MFMAs; two can hide each other's.
  constexpr int WAVES = ACT ? 8 : 4;
  constexpr int NTH = 64 * WAVES;
  constexpr int MT = ACT ? BM / 128 : 2;  // MFMA row tiles per wave
  int moe_row0 = 0;
  if constexpr (MOE) {
    moe_row0 = moe_enter(gp.p, gp.moe, blockIdx.y);
    if (gp.p.M <= 0) return;
  }
  constexpr bool TABLE = MODE == kModeActWide || MODE == kModeActNarrow;
  constexpr int GROUP_BYTES = MODE == kModeActWide ? kActWideGroupBytes : kActNarrowGroupBytes;
  constexpr int A_TILE = BM * kAUnits * 16;   // bytes
  constexpr int B_TILE = (kABK / 8) * kABN * 16;
  constexpr int A_LOADS = BM * (kABK / 8) / NTH;  // 16-byte activation loads per thread
  extern __shared__ __align__(16) unsigned char smem[];  // [A0][A1][B0][B1]
  const Problem& p = gp.p;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave >> 1, wn = wave & 1;
  const int j = lane & 31;
  const int kq = lane >> 5;
  const int N = p.N, K = p.K, M = p.M;
  const int NC = N >> 3;
  const int tiles_m = (M + BM - 1) / BM;
  const int tiles_all = tiles_m * (N / kABN);
  if constexpr (MOE) {
    if ((int)blockIdx.x >= tiles_all * gp.splits) return;
  }
  const int split = blockIdx.x / tiles_all;
  const int tile_id = blockIdx.x - split * tiles_all;
  const int tm = tile_id % tiles_m;
  const int tn = tile_id / tiles_m;
  const int m0 = tm * BM;
  const int n0 = tn * kABN;
  const int KT_all = K / kABK;
  const int kt_begin = (int)((long)split * KT_all / gp.splits);  // this workgroup's K tiles
  const int KT = (int)((long)(split + 1) * KT_all / gp.splits);
  const int last_tile = KT - 1;
  const AwqSplice splice = awq_splice_consts();

  // ---- producer state
  // AWQ: threads 0..127 own K block pb (8 rows) x word pc (8 columns).
  // act-order: wave w owns K block w (8 rows), its lane pq the two adjacent columns 2 pq, 2 pq + 1:
  // one 8-byte load fetches the two packed words and one LDS read per row the parameters of both
  // columns; the rows' groups are the same for the whole wave.
  const bool producer = ACT || tid < 128;
  const int pb = (tid >> 4) & 7;
  const int pc = tid & 15;
  const int pq = lane;
  const int pkb = wave;
  const uint32_t* wsrc = ACT ? p.qweight + (size_t)pkb * N + n0 + 2 * pq
                             : p.qweight + (size_t)(pb * 8) * NC + (n0 >> 3) + pc;
  uint32_t braw[8];  // AWQ: 8 rows of one word column
  uint4_t sraw;      // AWQ: 8 fp16 scales of the word's columns
  uint32_t zraw;     // AWQ: 8 zero-point nibbles
  // act-order: two register sets, the tile being unpacked and the one requested behind it
  uint2_t bw[2];     // packed words of the thread's two columns
  int gr[2][8];      // table modes: groups of the block's 8 rows
  auto load_b_act = [&](int kt, auto st_c) {
    constexpr int ST = decltype(st_c)::value;
    bw[ST] = *(const uint2_t*)(wsrc + (size_t)(kt * (kABK / 8)) * N);
    if constexpr (TABLE) {
      const int* gsrc = p.g_idx + kt * kABK + pkb * 8;
#pragma unroll
      for (int r = 0; r < 8; ++r) gr[ST][r] = gsrc[r];
    }
  };
  auto load_b = [&](int kt) {
    if (producer) {
#pragma unroll
      for (int r = 0; r < 8; ++r) braw[r] = wsrc[(size_t)(kt * kABK + r) * NC];
      const int g = min((kt * kABK + pb * 8) / p.groupsize, p.num_groups - 1);
      sraw = *(const uint4_t*)(p.scales + (size_t)g * N + n0 + pc * 8);
      zraw = p.qzeros[(size_t)g * NC + (n0 >> 3) + pc];
    }
  };
  const unsigned char* table = smem + 2 * A_TILE + 2 * B_TILE;  // act-order table modes only
  const int last_group = p.num_groups - 1;
  // The act-order producer works in three phases, so that the main loop can place MFMAs
  // between them.
  // Phase 1, once per tile: the parameters of the block's 8 rows for the two columns.  Wide
  // table: a[r][t] = scale | -(1024 + zero) << 16 of column t.  Otherwise a[r][0] = the two
  // fp16 scales, z[r] = the two zero points, one byte each.
  struct ActRows {
    uint32_t a[8][2];
    uint32_t z[8];
  };
  auto tile_params = [&](int kt, auto st_c, ActRows& ar) {
    constexpr int ST = decltype(st_c)::value;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      if constexpr (TABLE) {
        // a corrupt index stays inside the table
        const int g = min(max(gr[ST][r], 0), last_group);
        if constexpr (MODE == kModeActWide) {
          const uint2_t e = *(const uint2_t*)(table + g * GROUP_BYTES + 8 * pq);
          ar.a[r][0] = e.x; ar.a[r][1] = e.y;
        } else {
          ar.a[r][0] = *(const uint32_t*)(table + g * GROUP_BYTES + 4 * pq);
          ar.z[r] = *(const uint16_t*)(table + g * GROUP_BYTES + 2 * kABN + 2 * pq);
        }
      } else {
        int g = p.g_idx[kt * kABK + pkb * 8 + r];
        g = min(max(g, 0), last_group);
        ar.a[r][0] = *(const uint32_t*)(p.scales + (size_t)g * N + n0 + 2 * pq);
        // the word holds 8 columns: this thread's two are one byte of it
        const uint32_t zw = (gptq_zero_plus_one(p.qzeros[(size_t)g * NC + ((n0 + 2 * pq) >> 3)]) >> ((pq & 3) * 8)) & 0xFFu;
        ar.z[r] = (zw & 0xFu) | ((zw & 0xF0u) << 4);
      }
    }
  };
  // Phase 2: rows pr and pr + 4 of column t share one splice (their nibbles sit 16 bits apart).
  auto word_pair = [&](uint32_t w, auto t_c, int pr, const ActRows& ar) -> uint32_t {
    constexpr int T = decltype(t_c)::value;
    const uint32_t q2 = ((w >> (4 * pr)) & splice.mask_lo) | splice.magic;
    uint32_t s2, cz2;
    if constexpr (MODE == kModeActWide) {
      s2 = __builtin_amdgcn_perm(ar.a[pr + 4][T], ar.a[pr][T], 0x05040100u);
      cz2 = __builtin_amdgcn_perm(ar.a[pr + 4][T], ar.a[pr][T], 0x07060302u);
    } else {
      s2 = __builtin_amdgcn_perm(ar.a[pr + 4][0], ar.a[pr][0], (T & 1) ? 0x07060302u : 0x05040100u);
      cz2 = 0xE400E400u | __builtin_amdgcn_perm(ar.z[pr + 4], ar.z[pr], 0x0C000C00u | (uint32_t)T | ((uint32_t)(4 + T) << 16));
    }
    const half2_t dq = as_half2(q2) + as_half2(cz2);  // exact q - z
    if constexpr (DTYPE == Q4_DTYPE_F16) {
      return as_u32(dq * as_half2(s2));  // one fp16 rounding
    } else {
      // bf16: the exact fp32 product, one mixed-precision multiply per weight straight from the
      // fp16 halves (the compiler would emit two converts and a multiply), rounded once
      const uint32_t dqu = as_u32(dq);
      awq_float2_t f;
      asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[0,0,0] op_sel_hi:[1,1,0]" : "=v"(f.x) : "v"(dqu), "v"(s2));
      asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,1,0] op_sel_hi:[1,1,0]" : "=v"(f.y) : "v"(dqu), "v"(s2));
      return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, awq_bf16x2_t));
    }
  };
  // Phase 3: o holds rows (0,4),(1,5),(2,6),(3,7) of column t: back to natural K order, one
  // 16-byte unit.
  auto word_store = [&](int buf, int t, const uint32_t (&o)[4]) {
    unsigned char* base = smem + 2 * A_TILE + buf * B_TILE;
    uint4_t unit;  // one byte permute per register
    unit.x = __builtin_amdgcn_perm(o[1], o[0], 0x05040100u);
    unit.y = __builtin_amdgcn_perm(o[3], o[2], 0x05040100u);
    unit.z = __builtin_amdgcn_perm(o[1], o[0], 0x07060302u);
    unit.w = __builtin_amdgcn_perm(o[3], o[2], 0x07060302u);
    *(uint4_t*)(base + ((size_t)pkb * kABN + b_slot(2 * pq + t)) * 16) = unit;
  };
  auto word_of = [&](const uint2_t& w, int t) { return t == 0 ? w.x : w.y; };
  // whole tile at once (prologue only)
  auto store_b_act = [&](int buf, int kt, auto st_c) {
    constexpr int ST = decltype(st_c)::value;
    ActRows ar;
    tile_params(kt, st_c, ar);
    auto one = [&](auto t_c) {
      constexpr int T = decltype(t_c)::value;
      uint32_t o[4];
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) o[pr] = word_pair(word_of(bw[ST], T), t_c, pr, ar);
      word_store(buf, T, o);
    };
    one(std::integral_constant<int, 0>{});
    one(std::integral_constant<int, 1>{});
  };
  auto store_b_awq = [&](int buf) {
    if (!producer) return;
    unsigned char* base = smem + 2 * A_TILE + buf * B_TILE;
    const uint32_t su[4] = {sraw.x, sraw.y, sraw.z, sraw.w};
    const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
    half2_t d[8][4];  // [nibble position][row pair]: exact q - z
#pragma unroll
    for (int rp = 0; rp < 4; ++rp) {
#pragma unroll
      for (int by = 0; by < 4; ++by) {
        const uint32_t sel = 0x0C000C00u | (uint32_t)by | ((uint32_t)(4 + by) << 16);
        const uint32_t t2 = __builtin_amdgcn_perm(braw[2 * rp + 1], braw[2 * rp], sel);
        const uint32_t ze = (zraw >> (8 * by)) & 0xFu;       // position 2*by
        const uint32_t zo = (zraw >> (8 * by + 4)) & 0xFu;   // position 2*by + 1
        d[2 * by][rp] = as_half2((t2 & splice.mask_lo) | splice.magic) +
                        as_half2(0xE400E400u | ze | (ze << 16));
        d[2 * by + 1][rp] = as_half2((t2 & splice.mask_hi) | splice.magic) * sixteenth +
                            as_half2(0xD400D400u | (zo << 4) | (zo << 20));
      }
    }
#pragma unroll
    for (int pos = 0; pos < 8; ++pos) {
      const int col = ((pos & 3) << 1) | (pos >> 2);  // logical column of this nibble position
      const half2_t pr = as_half2(su[col >> 1]);
      const half_t s = (col & 1) ? pr.y : pr.x;
      uint4_t unit;
      uint32_t o[4];
#pragma unroll
      for (int rp = 0; rp < 4; ++rp) {
        if constexpr (DTYPE == Q4_DTYPE_F16) {
          o[rp] = as_u32(d[pos][rp] * half2_t{s, s});  // one fp16 rounding per weight
        } else {
          const awq_float2_t f = {(float)d[pos][rp].x * (float)s, (float)d[pos][rp].y * (float)s};
          o[rp] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, awq_bf16x2_t));
        }
      }
      unit.x = o[0]; unit.y = o[1]; unit.z = o[2]; unit.w = o[3];
      *(uint4_t*)(base + ((size_t)pb * kABN + b_slot(pc * 8 + col)) * 16) = unit;
    }
  };


  // ---- activation tile: global -> registers -> LDS (natural K order)
  const uint16_t* xs = (const uint16_t*)p.x;
  uint4_t areg[A_LOADS];
  int moe_xrow[MOE ? A_LOADS : 1];  // grouped launch with a row map: x row of each staged row
  if constexpr (MOE) {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int row = min(m0 + ((tid + NTH * i) >> 3), M - 1);
      moe_xrow[i] = gp.moe.x_rows != nullptr ? gp.moe.x_rows[moe_row0 + row] : row;
    }
  }
  auto load_a = [&](int kt) {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + NTH * i;
      const int m = u >> 3, kb = u & 7;
      // rows past M re-read the last row, never stored
      const int row = MOE ? moe_xrow[i] : min(m0 + m, M - 1);
      areg[i] = *(const uint4_t*)(xs + (size_t)row * K + kt * kABK + kb * 8);
    }
  };
  auto store_a = [&](int buf) {
    unsigned char* base = smem + buf * A_TILE;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + NTH * i;
      const int m = u >> 3, kb = u & 7;
      *(uint4_t*)(base + (m * kAUnits + kb) * 16) = areg[i];
    }
  };

  float16_t acc[MT][2];
#pragma unroll
  for (int a = 0; a < MT; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  if constexpr (TABLE) {
    // every group's parameters for this tile's 128 columns: 16 scale units + 16 zero words each
    unsigned char* tab = smem + 2 * A_TILE + 2 * B_TILE;
    for (int u = tid; u < p.num_groups * 16; u += NTH) {
      const int g = u >> 4, c = u & 15;
      const uint4_t s8 = *(const uint4_t*)(p.scales + (size_t)g * N + n0 + c * 8);
      const uint32_t zw = gptq_zero_plus_one(p.qzeros[(size_t)g * NC + (n0 >> 3) + c]);
      if constexpr (MODE == kModeActWide) {
        const uint32_t sp[4] = {s8.x, s8.y, s8.z, s8.w};
        uint32_t e[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
          const uint32_t sbits = (q & 1) ? sp[q >> 1] >> 16 : sp[q >> 1] & 0xFFFFu;
          e[q] = sbits | ((0xE400u | ((zw >> (4 * q)) & 0xFu)) << 16);
        }
        uint4_t* dst = (uint4_t*)(tab + g * GROUP_BYTES + c * 32);
        dst[0] = uint4_t{e[0], e[1], e[2], e[3]};
        dst[1] = uint4_t{e[4], e[5], e[6], e[7]};
      } else {
        uint2_t zb;  // one byte per zero point, column order
        zb.x = (zw & 0xFu) | ((zw & 0xF0u) << 4) | ((zw & 0xF00u) << 8) | ((zw & 0xF000u) << 12);
        zb.y = ((zw >> 16) & 0xFu) | ((zw >> 12) & 0xF00u) | ((zw >> 8) & 0xF0000u) | ((zw >> 4) & 0xF000000u);
        *(uint4_t*)(tab + g * GROUP_BYTES + c * 16) = s8;
        *(uint2_t*)(tab + g * GROUP_BYTES + 2 * kABN + c * 8) = zb;
      }
    }
    __syncthreads();
  }
  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  load_a(kt_begin);
  if constexpr (ACT) {
    // set 1 takes the first tile, set 0 the second: iteration i of the loop unpacks set i & 1
    load_b_act(kt_begin, I1{});
    load_b_act(min(kt_begin + 1, last_tile), I0{});
    store_a(0);
    store_b_act(0, kt_begin, I1{});
  } else {
    load_b(kt_begin);
    store_a(0);
    store_b_awq(0);
    load_b(min(kt_begin + 1, last_tile));
  }
  load_a(min(kt_begin + 1, last_tile));
  __syncthreads();

  const int a_off = ((wm * 32 * MT + j) * kAUnits + kq) * 16;
  const int b_off[2] = {(kq * kABN + b_slot(wn * 64 + j)) * 16, (kq * kABN + b_slot(wn * 64 + 32 + j)) * 16};

  auto read_frags = [&](const unsigned char* ab, const unsigned char* bb, int s, uint4_t (&af)[MT], uint4_t (&bf)[2]) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) af[mt] = *(const uint4_t*)(ab + (mt * 32 * kAUnits + 2 * s) * 16);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) bf[nt] = *(const uint4_t*)(bb + b_off[nt] + (2 * s) * kABN * 16);
  };
  auto mfma_one = [&](const uint4_t& a, const uint4_t& b, float16_t& c) {
    if constexpr (DTYPE == Q4_DTYPE_F16) {
      c = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, b), c, 0, 0, 0);
    } else {
      c = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
  };
  auto mfma_frags = [&](const uint4_t (&af)[MT], const uint4_t (&bf)[2]) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) mfma_one(af[mt], bf[nt], acc[mt][nt]);
  };
  auto mfma_step = [&](const unsigned char* ab, const unsigned char* bb, int s) {
    uint4_t af[MT], bf[2];
    read_frags(ab, bb, s, af, bf);
    mfma_frags(af, bf);
  };

  // One K tile.  ST: the act-order register set that holds the next tile's packed words (also
  // the parity of the LDS buffer being multiplied).
  auto tile_step = [&](int kt, auto st_c) {
    constexpr int ST = decltype(st_c)::value;
    const int cur = (kt - kt_begin) & 1;
    const int kt1 = min(kt + 1, last_tile);
    const int kt2 = min(kt + 2, last_tile);
    const unsigned char* ab = smem + cur * A_TILE + a_off;
    const unsigned char* bb = smem + 2 * A_TILE + cur * B_TILE;
    // the other buffer was last read in tile kt-1, before the barrier that ended it
    store_a(cur ^ 1);
    load_a(kt2);
    if constexpr (ACT) {
      // the set unpacked in the previous tile is free: request the tile after the next
      load_b_act(kt2, std::integral_constant<int, ST ^ 1>{});
      // the next tile's parameters first, then half a column (two row pairs) per MFMA K step,
      // unpacked in phases with this tile's MFMAs between them (the order is pinned)
      static_assert(kABK / 16 == 4, "half a producer column per MFMA K step");
      ActRows ar;
      // fragments one K step ahead
      uint4_t af[2][MT], bf[2][2];
      uint32_t o[4];
      tile_params(kt1, st_c, ar);
      read_frags(ab, bb, 0, af[0], bf[0]);
      auto step = [&](auto s_c) {
        constexpr int S = decltype(s_c)::value;
        constexpr int P = S & 1;
        constexpr int H = S & 1;  // which two row pairs of the column
        using T = std::integral_constant<int, (S >> 1)>;
        if constexpr (S < 3) read_frags(ab, bb, S + 1, af[P ^ 1], bf[P ^ 1]);
        const uint32_t w = word_of(bw[ST], S >> 1);
        __builtin_amdgcn_sched_barrier(0);
        mfma_one(af[P][0], bf[P][0], acc[0][0]);
        __builtin_amdgcn_sched_barrier(0);
        o[2 * H] = word_pair(w, T{}, 2 * H, ar);
        o[2 * H + 1] = word_pair(w, T{}, 2 * H + 1, ar);
        __builtin_amdgcn_sched_barrier(0);
        mfma_one(af[P][0], bf[P][1], acc[0][1]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (H == 1) word_store(cur ^ 1, S >> 1, o);
        if constexpr (MT == 2) {
          __builtin_amdgcn_sched_barrier(0);
          mfma_one(af[P][1], bf[P][0], acc[1][0]);
          mfma_one(af[P][1], bf[P][1], acc[1][1]);
          __builtin_amdgcn_sched_barrier(0);
        }
      };
      step(std::integral_constant<int, 0>{});
      step(std::integral_constant<int, 1>{});
      step(std::integral_constant<int, 2>{});
      step(std::integral_constant<int, 3>{});
    } else {
      store_b_awq(cur ^ 1);
      load_b(kt2);
#pragma unroll
      for (int s = 0; s < kABK / 16; ++s) mfma_step(ab, bb, s);
    }
    __syncthreads();
  };
  for (int kt = kt_begin; kt < KT; kt += 2) {
    tile_step(kt, I0{});
    if (kt + 1 < KT) tile_step(kt + 1, I1{});
  }

  // ---- epilogue: register r of lane (j, kq) is row 8*(r/4) + 4*kq + r%4, column j
  if (gp.splits > 1) {
    float* part = gp.partials + ((size_t)split * gp.partial_rows + moe_row0) * N;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int n = n0 + wn * 64 + nt * 32 + j;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * 32 * MT + mt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
          if (m < M) part[(size_t)m * N + n] = acc[mt][nt][r];
        }
      }
    }
    return;
  }
  uint16_t* y = (uint16_t*)p.y;
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int n = n0 + wn * 64 + nt * 32 + j;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 32 * MT + mt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
        if (m < M) y[(size_t)m * N + n] = finish_output<DTYPE>(acc[mt][nt][r], p.bias, n);
      }
    }
  }
}

}  // namespace q4

namespace q4host {

bool gemm_awq_supported(const q4_weight* w, int M, int dtype) {
  (void)dtype;
  if (M < 1) return false;
  if (w->K % q4::kABK != 0 || w->N % q4::kABN != 0) return false;
  if (w->layout == Q4_LAYOUT_GPTQ) return w->g_idx != nullptr;  // act-order
  // AWQ: one group per 8-row K block
  if (w->groupsize % 8 != 0) return false;
  return (long)w->num_groups * w->groupsize >= w->K;
}

constexpr size_t kAwqTilesLdsBytes = 2 * (size_t)q4::kABM * q4::kAUnits * 16 + 2 * (size_t)(q4::kABK / 8) * q4::kABN * 16;
// with 256-row tiles (act-order, table modes)
constexpr size_t kActTallTilesLdsBytes = 4 * (size_t)q4::kABM * q4::kAUnits * 16 + 2 * (size_t)(q4::kABK / 8) * q4::kABN * 16;

// Kernel variant for a weight: act-order takes the 32-bit parameter table where it fits
// beside the tiles, except that the smaller table is taken when only it leaves room for two
// workgroups per CU and the grid has more than one workgroup per CU to offer; layers with
// too many groups for either table gather from global memory.
static int gemm_awq_mode(const q4_weight* w, long workgroups, size_t tiles_bytes = kAwqTilesLdsBytes) {
  using namespace q4;
  if (w->layout != Q4_LAYOUT_GPTQ) return kModeAwq;
  const size_t wide = tiles_bytes + (size_t)w->num_groups * kActWideGroupBytes;
  const size_t narrow = tiles_bytes + (size_t)w->num_groups * kActNarrowGroupBytes;
  const bool narrow_doubles =
      workgroups > 256 && wide > kLdsBytesPerWorkgroup / 2 && narrow <= kLdsBytesPerWorkgroup / 2;
  if (wide <= kLdsBytesPerWorkgroup && !narrow_doubles) return kModeActWide;
  if (narrow <= kLdsBytesPerWorkgroup) return kModeActNarrow;
  return kModeActGather;
}

bool gemm_act_order_table(const q4_weight* w) {
  return w->layout == Q4_LAYOUT_GPTQ && w->g_idx != nullptr && gemm_awq_mode(w, 0) != q4::kModeActGather;
}

// 128 x 128 tiles, ~1.0 us per K tile alone on a CU, ~1.9 us when two workgroups share it.
// one_per_cu: act-order with its parameter table in LDS, which leaves room for a single
// workgroup per CU (~1.0 us per K tile).  There a grid of a few hundred tiles runs in
// rounds of 256 and a last, mostly empty round costs as much as a full one, so split-K is
// also weighed above 256 tiles (8192 x 10240 at M = 512: 320 tiles, 2 rounds).
// Act-order with its table in LDS, dense launches: 256-row tiles (the unpacked weight tile serves
// twice the rows; a K tile takes about 1.5x as long) where they fit beside the table and the
// estimate below, rounds of 256 workgroups and split-K included, is the shorter one.  Measured on
// MI355X, 256- against 128-row tiles (us): 8192 x 10240 158 / 201 at M = 512, 302 / 345 at M = 1024,
// 493 / 558 at M = 2048, 846 / 1067 at M = 4096, but 162 / 137 at M = 384; 4096 x 14336 88 / 101 at
// M = 512, 177 / 201 at M = 1024, but 169 / 152 at M = 768.
// estimated time (us) of a dense act-order launch with one workgroup per CU: the split-K cost
// model of gemm_pick_splits with the measured time of a K tile (0.85 us at 128 rows, 1.28 us at 256)
static double act_estimate_us(int M, int K, int N, int bm, double us_tile) {
  static const int kCandidates[] = {1, 2, 3, 4, 6, 8, 12, 16};
  const long tiles = (long)((M + bm - 1) / bm) * (N / q4::kABN);
  const int KT = K / q4::kABK;
  double best = -1.0;
  for (int sp : kCandidates) {
    if (sp > 1 && (KT / sp < 8 || tiles >= 1024)) break;
    double t = (double)((tiles * sp + 255) / 256) * ((KT + sp - 1) / sp) * us_tile;
    if (sp > 1) t += 5.0 + (double)sp * M * N * 8.0 / 5.0e6;
    if (best < 0.0 || t < best) best = t;
  }
  return best;
}
bool gemm_act_order_tall(const q4_weight* w, int M) {
  // (below 512 rows the launches are split-K heavy and the estimate is not good enough to choose)
  if (w->layout != Q4_LAYOUT_GPTQ || w->g_idx == nullptr || M < 4 * q4::kABM) return false;
  if (kActTallTilesLdsBytes + (size_t)w->num_groups * q4::kActNarrowGroupBytes > q4::kLdsBytesPerWorkgroup) return false;
  return act_estimate_us(M, w->K, w->N, 2 * q4::kABM, 1.28) < 0.95 * act_estimate_us(M, w->K, w->N, q4::kABM, 0.85);
}

int gemm_awq_splits(int M, int K, int N, bool one_per_cu, bool tall) {
  if (K % q4::kABK != 0 || N % q4::kABN != 0) return 1;
  const int bm = tall ? 2 * q4::kABM : q4::kABM;
  const long tiles = (long)((M + bm - 1) / bm) * (N / q4::kABN);
  if (one_per_cu) return tiles < 1024 ? gemm_pick_splits(tiles, K / q4::kABK, M, N, 1.0, 1.0, 1) : 1;
  return tiles < 256 ? gemm_pick_splits(tiles, K / q4::kABK, M, N, 1.0, 1.9) : 1;
}

// Split-K factor of a grouped launch.  The host does not know the experts' row counts: it
// plans for an even spread (pairs / experts rows each).
static int moe_awq_splits(const q4_weight* w, const MoeLaunch* moe) {
  const long avg_rows = ((long)moe->pairs + moe->num_experts - 1) / moe->num_experts;
  const long tiles = (long)moe->num_experts * ((avg_rows + q4::kABM - 1) / q4::kABM) * (w->N / q4::kABN);
  if (gemm_act_order_table(w)) return tiles < 1024 ? gemm_pick_splits(tiles, w->K / q4::kABK, moe->pairs, w->N, 1.0, 1.0, 1) : 1;
  return tiles < 256 ? gemm_pick_splits(tiles, w->K / q4::kABK, moe->pairs, w->N, 1.0, 1.9) : 1;
}

size_t gemm_awq_moe_workspace_bytes(const q4_weight* w, const MoeLaunch* moe) {
  const int splits = moe_awq_splits(w, moe);
  return splits > 1 ? (size_t)splits * moe->pairs * w->N * sizeof(float) : 0;
}

int launch_gemm_awq(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                    void* workspace, size_t workspace_bytes, hipStream_t stream, const MoeLaunch* moe) {
  using namespace q4;
  // dense AWQ launches go to the kernel that unpacks the words in registers where it applies
  if (moe == nullptr && gemm_awq_direct_supported(w, M, dtype))
    return launch_gemm_awq_direct(w, x, bias, y, M, dtype, workspace, workspace_bytes, stream);
  // grouped launch: M is the largest row count an expert can have (the number of tokens)
  if (!gemm_awq_supported(w, M, dtype)) {
    set_error("q4_linear(gemm/awq): unsupported problem (M=%d K=%d N=%d groupsize=%d)", M, w->K, w->N,
              w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  AwqGemmParams gp;
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, w->g_idx, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  const int out_rows = moe != nullptr ? moe->pairs : M;  // rows of y (and of one split's partials)
  const bool tall = moe == nullptr && gemm_act_order_tall(w, M);
  const int bm = tall ? 2 * kABM : kABM;
  int splits = moe != nullptr ? moe_awq_splits(w, moe) : gemm_awq_splits(M, w->K, w->N, gemm_act_order_table(w), tall);
  if (splits > 1 && (workspace == nullptr ||
                     workspace_bytes < Q4_WORKSPACE_COUNTER_BYTES + (size_t)splits * out_rows * w->N * sizeof(float)))
    splits = 1;  // no room for partial tiles: one workgroup per whole tile
  gp.splits = splits;
  gp.partial_rows = out_rows;
  gp.partials = splits > 1 ? (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES) : nullptr;
  gp.moe = moe != nullptr ? moe->view : MoeView{};
  const long total = (long)((M + bm - 1) / bm) * (w->N / kABN) * splits;
  const long experts = moe != nullptr ? moe->num_experts : 1;
  if (total > 0x7fffffffL || experts > 65535) {
    set_error("q4_linear(gemm/awq): grid too large");
    return Q4_ERR_UNSUPPORTED;
  }
  const size_t tiles_smem = tall ? kActTallTilesLdsBytes : kAwqTilesLdsBytes;
  const int mode = gemm_awq_mode(w, total * experts, tiles_smem);
  const size_t smem = tiles_smem + (mode == kModeActWide     ? (size_t)w->num_groups * kActWideGroupBytes
                                    : mode == kModeActNarrow ? (size_t)w->num_groups * kActNarrowGroupBytes
                                                             : 0);
  const dim3 grid((unsigned)total, (unsigned)experts);
  auto launch = [&](auto k) {
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(mode == kModeAwq ? 256 : 512), smem, stream, gp);
  };
  auto launch_mode = [&](auto dt, auto grouped) {
    constexpr int DT = decltype(dt)::value;
    constexpr bool G = decltype(grouped)::value;
    if constexpr (!G) {
      if (tall) {
        if (mode == kModeActWide) launch(gemm_awq_kernel<DT, kModeActWide, false, 2 * kABM>);
        else launch(gemm_awq_kernel<DT, kModeActNarrow, false, 2 * kABM>);
        return;
      }
    }
    switch (mode) {
      case kModeAwq: launch(gemm_awq_kernel<DT, kModeAwq, G>); break;
      case kModeActWide: launch(gemm_awq_kernel<DT, kModeActWide, G>); break;
      case kModeActNarrow: launch(gemm_awq_kernel<DT, kModeActNarrow, G>); break;
      default: launch(gemm_awq_kernel<DT, kModeActGather, G>); break;
    }
  };
  using F16 = std::integral_constant<int, Q4_DTYPE_F16>;
  using BF16 = std::integral_constant<int, Q4_DTYPE_BF16>;
  if (moe != nullptr) {
    if (dtype == Q4_DTYPE_F16) launch_mode(F16{}, std::true_type{});
    else launch_mode(BF16{}, std::true_type{});
  } else {
    if (dtype == Q4_DTYPE_F16) launch_mode(F16{}, std::false_type{});
    else launch_mode(BF16{}, std::false_type{});
  }
  if (splits > 1) launch_gemm_reduce(gp.partials, bias, y, out_rows, w->N, splits, dtype, stream);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemm/awq): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
