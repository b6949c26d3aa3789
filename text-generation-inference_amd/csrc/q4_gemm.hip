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
};

typedef float float2_t __attribute__((ext_vector_type(2)));

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
  float sf;            // float(s), bf16 path
};

__device__ __forceinline__ ColConsts make_col_consts(uint32_t z, half_t s) {
  ColConsts c;
  c.czlo = as_half2(0xE400E400u | z | (z << 16));
  c.czhi = as_half2(0xD400D400u | (z << 4) | (z << 20));
  c.s2 = half2_t{s, s};
  c.sf = (float)s;
  return c;
}

// One packed word -> MFMA B fragment (8 weights of one column, K order 0,4,1,5,2,6,3,7).
template <int DTYPE>
__device__ __forceinline__ uint4_t dequant_word(uint32_t w, const ColConsts& c, const SpliceK& k) {
  const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
  const uint32_t w8 = w >> 8;
  half2_t d[4];  // exact (q - z)
  d[0] = as_half2((w & k.mask_lo) | k.magic) + c.czlo;
  d[1] = as_half2((w & k.mask_hi) | k.magic) * sixteenth + c.czhi;
  d[2] = as_half2((w8 & k.mask_lo) | k.magic) + c.czlo;
  d[3] = as_half2((w8 & k.mask_hi) | k.magic) * sixteenth + c.czhi;
  uint4_t out;
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    // one fp16 multiply per weight: the reference's rounding
    out.x = as_u32(d[0] * c.s2);
    out.y = as_u32(d[1] * c.s2);
    out.z = as_u32(d[2] * c.s2);
    out.w = as_u32(d[3] * c.s2);
  } else {
    // bf16: exact fp32 product, rounded once
    uint32_t o[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float lo = (float)d[i].x * c.sf;
      const float hi = (float)d[i].y * c.sf;
      o[i] = (uint32_t)f32_to_bf16_rne(lo) | ((uint32_t)f32_to_bf16_rne(hi) << 16);
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

// BM: rows per workgroup (128 or 256).  GPT: quantisation groups per K tile (1 or 2).
// NW: packed words (columns) per lane and K step: 2 -> 256-column workgroup tile, 1 -> 128.
template <int DTYPE, int BM, int GPT, int NW>
__global__ __launch_bounds__(256, (BM == 128 ? (NW == 1 ? 3 : 2) : 1)) void gemm_gptq_kernel(GemmParams gp) {
  constexpr int MT = BM / 32;                      // MFMA row tiles per wave
  constexpr int A_LOADS = BM * (kBK / 8) / 256;    // 16-byte activation loads per thread per tile
  constexpr int A_TILE_BYTES = BM * kAUnitsPerRow * 16;
  extern __shared__ __align__(16) unsigned char smem[];  // two activation tiles
  const Problem& p = gp.p;
  const int tid = threadIdx.x;
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
  const int nw = n0 + wave * 32 * NW;  // first column of this wave
  const int ncol = nw + NW * j;        // first of this lane's NW columns

  const SpliceK splice = gemm_splice_consts();
  const int KT_all = K / kBK;
  // this workgroup's K tiles [kt_begin, KT)
  const int kt_begin = (int)((long)split * KT_all / gp.splits);
  const int KT = (int)((long)(split + 1) * KT_all / gp.splits);

  // ---- packed-weight stream: words [K/8 + kq][ncol, ncol+1], two K tiles ahead
  const char* wbase = (const char*)p.qweight;
  const uint32_t w_lane = ((uint32_t)kq * (uint32_t)N + (uint32_t)ncol) * 4u;
  const size_t kstep_bytes = (size_t)N * 8;  // two packed rows per MFMA K step
  struct BWords { uint32_t v[NW]; };
  BWords bq[2][kKSteps];
  auto load_b = [&](int kt, BWords (&dst)[kKSteps]) {
#pragma unroll
    for (int s = 0; s < kKSteps; ++s)
    {
      const char* addr = wbase + (size_t)(kt * kKSteps + s) * kstep_bytes + w_lane;
      if constexpr (NW == 2) {
        const uint2_t t = *(const uint2_t*)addr;
        dst[s].v[0] = t.x; dst[s].v[1] = t.y;
      } else {
        dst[s].v[0] = *(const uint32_t*)addr;
      }
    }
  };

  // ---- group constants for this lane's two columns.  They are rebuilt for every tile
  // from two tiny (cached) loads, which keeps the steady-state loop free of branches.
  ColConsts cc[GPT][NW], cc_next[GPT][NW];
  uint32_t sraw[GPT], zraw[GPT];
  const int zshift = (ncol & 7) * 4;
  auto load_group_raw = [&](int kt) {
#pragma unroll
    for (int g = 0; g < GPT; ++g) {
      int gi = (kt * kBK + g * (kBK / GPT)) / p.groupsize;
      gi = min(gi, p.num_groups - 1);
      if constexpr (NW == 2) sraw[g] = *(const uint32_t*)(p.scales + (size_t)gi * N + ncol);
      else sraw[g] = *(const uint16_t*)(p.scales + (size_t)gi * N + ncol);
      zraw[g] = p.qzeros[(size_t)gi * (N >> 3) + (ncol >> 3)];
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
  const uint16_t* xs = (const uint16_t*)p.x;
  // Register staging sets: with two sets (128-row tiles) a tile's loads are issued two
  // tiles before they are written to LDS; the 256-row tile has registers for one set only.
  constexpr int ASETS = BM == 128 ? 2 : 1;
  uint4_t areg[ASETS][A_LOADS];
  auto load_a = [&](int kt, auto set_c) {
    constexpr int set = decltype(set_c)::value % ASETS;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + 256 * i;
      const int m = u >> 3, kb = u & 7;
      // rows past M re-read the last row: their results are never stored
      const int row = min(m0 + m, M - 1);
      areg[set][i] = *(const uint4_t*)(xs + (size_t)row * K + kt * kBK + kb * 8);
    }
  };
  auto store_a = [&](int buf, auto set_c) {
    constexpr int set = decltype(set_c)::value % ASETS;
    unsigned char* base = smem + buf * A_TILE_BYTES;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + 256 * i;
      const int m = u >> 3, kb = u & 7;
      const uint4_t v = areg[set][i];
      uint4_t o;
      o.x = (v.x & 0xFFFFu) | (v.z << 16);
      o.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
      o.z = (v.y & 0xFFFFu) | (v.w << 16);
      o.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
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
    const unsigned char* abase = smem + buf * A_TILE_BYTES + a_lane_off;
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

  // ---- epilogue: C layout of the 32x32 MFMA: register r of lane (j, kq) is row
  // 8*(r/4) + 4*kq + r%4, column j.  Fragments 0/1 are adjacent columns -> one 32-bit store.
  if (gp.splits > 1) {
    // fp32 partial tile; bias, rounding and the store to y happen in the reduction kernel
    float* part = gp.partials + (size_t)split * M * N;
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
    float4_t sum = *(const float4_t*)(partials + e);
    for (int sp = 1; sp < splits; ++sp) {
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

namespace q4host {

using q4::GemmParams;
using q4::Problem;

bool gemm_supported(const q4_weight* w, int M, int dtype) {
  (void)dtype;
  if (w->layout != Q4_LAYOUT_GPTQ || w->g_idx != nullptr) return false;
  if (M < 1) return false;
  if (w->K % q4::kBK != 0 || w->N % 128 != 0) return false;
  const int gs = w->groupsize;
  if (!(gs == 32 || (gs >= 64 && gs % 64 == 0))) return false;
  if ((long)w->num_groups * gs < w->K) return false;
  return true;
}

template <int DTYPE, int BM, int NW>
static void launch_tile(const GemmParams& gp, int gs, dim3 grid, size_t smem, hipStream_t stream) {
  using namespace q4;
  if (gs == 32) {
    auto k = gemm_gptq_kernel<DTYPE, BM, 2, NW>;
    if (smem > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(256), smem, stream, gp);
  } else {
    auto k = gemm_gptq_kernel<DTYPE, BM, 1, NW>;
    if (smem > 64 * 1024)
      (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, grid, dim3(256), smem, stream, gp);
  }
}

// Tile shape and split factor for a problem; shared by the launcher and the workspace sizing.
struct GemmPlan {
  int bm, nw, splits;
  long tiles;
};

static GemmPlan gemm_plan(int M, int K, int N) {
  // Tile choice (all with 4 waves side by side along N):
  //   256 x 256  grids of at least two rounds over the 256 CUs: half the unpacking per flop,
  //              one wave per SIMD, runs at a higher clock;
  //   128 x 256  the default; two workgroups per CU once there are more than 256 of them;
  //   128 x 128  only when N is not a multiple of 256 (measured slower than 128 x 256
  //              everywhere else: twice the activation-fragment reads per MFMA).
  GemmPlan g;
  const bool n256 = N % 256 == 0;
  const long t256 = n256 ? (long)((M + 255) / 256) * (N / 256) : 0;
  g.bm = 128;
  g.nw = n256 ? 2 : 1;
  if (t256 >= 512) g.bm = 256;
  const int bn = 128 * g.nw;
  g.tiles = (long)((M + g.bm - 1) / g.bm) * (N / bn);
  // Split-K when the tiles alone leave CUs idle (one workgroup runs the whole K loop at
  // ~0.9 us per 64-row K tile whatever M is: 14336 x 4096 took 200 us for every M up to
  // 1024).  Aim at two workgroups per CU, keep at least 8 K tiles per workgroup.
  // The split factor minimises a cost model fitted to measurements on MI355X: a workgroup
  // takes ~0.9 us per K tile alone on its CU and ~1.3 us when two share one; the partial
  // tiles cost a second launch (~5 us) plus S * M * N * 8 bytes of traffic at ~5 TB/s.
  // (4096 x 6144 at M = 1024: 70 us unsplit, 86 us with three splits; 14336 x 4096 at
  // M = 512: 200 us unsplit, 78 us with eight.)
  g.splits = 1;
  if (g.bm == 128 && g.tiles < 256) g.splits = gemm_pick_splits(g.tiles, K / q4::kBK, M, N, 0.9, 1.3);
  return g;
}

// per_cu: workgroups of this kernel that fit on a CU together (1 or 2)
int gemm_pick_splits(long tiles, int KT, int M, int N, double us_alone, double us_shared, int per_cu) {
  static const int kCandidates[] = {1, 2, 3, 4, 6, 8, 12, 16};
  double best = -1.0;
  int splits = 1;
  for (int sp : kCandidates) {
    if (sp > 1 && KT / sp < 8) break;  // at least 8 K tiles (512 rows) per workgroup
    const long wgs = tiles * sp;
    const long slots = 256L * per_cu;
    const long rounds = (wgs + slots - 1) / slots;
    const double per_tile = (per_cu == 1 || wgs <= 256) ? us_alone : us_shared;
    double t = (double)rounds * ((KT + sp - 1) / sp) * per_tile;
    if (sp > 1) t += 5.0 + (double)sp * M * N * 8.0 / 5.0e6;
    if (best < 0.0 || t < best) {
      best = t;
      splits = sp;
    }
  }
  return splits;
}

void launch_gemm_reduce(const float* partials, const void* bias, void* y, int M, int N, int splits, int dtype,
                        hipStream_t stream) {
  const long quads = (long)M * (N / 4);
  long blocks = (quads + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  if (dtype == Q4_DTYPE_F16)
    hipLaunchKernelGGL(q4::gemm_reduce_kernel<Q4_DTYPE_F16>, dim3((unsigned)blocks), dim3(256), 0, stream, partials,
                       bias, (uint16_t*)y, M, N, splits);
  else
    hipLaunchKernelGGL(q4::gemm_reduce_kernel<Q4_DTYPE_BF16>, dim3((unsigned)blocks), dim3(256), 0, stream, partials,
                       bias, (uint16_t*)y, M, N, splits);
}

// fp32 partial tiles of the split-K variants: splits x M x N floats (upper bound over the
// GPTQ kernel and the AWQ / act-order kernel, whose tiles differ).
size_t gemm_workspace_bytes(int M, int K, int N) {
  if (M <= 16 || K % q4::kBK != 0 || N % 128 != 0) return 0;
  int splits = gemm_plan(M, K, N).splits;
  for (const bool one_per_cu : {false, true}) {
    const int other = gemm_awq_splits(M, K, N, one_per_cu);
    if (other > splits) splits = other;
  }
  return splits > 1 ? (size_t)splits * M * N * sizeof(float) : 0;
}

int launch_gemm(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                void* workspace, size_t workspace_bytes, hipStream_t stream) {
  using namespace q4;
  if (!gemm_supported(w, M, dtype)) {
    set_error("q4_linear(gemm): unsupported problem (layout=%d g_idx=%p M=%d K=%d N=%d groupsize=%d)",
              w->layout, (const void*)w->g_idx, M, w->K, w->N, w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  GemmParams gp;
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, nullptr, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  GemmPlan g = gemm_plan(M, w->K, w->N);
  // without room for the partial tiles every workgroup owns a whole tile (slower, same result
  // up to fp32 summation order)
  const size_t partial_bytes = (size_t)g.splits * M * w->N * sizeof(float);
  if (g.splits > 1 && (workspace == nullptr || workspace_bytes < Q4_WORKSPACE_COUNTER_BYTES + partial_bytes))
    g.splits = 1;
  gp.splits = g.splits;
  gp.partials = g.splits > 1 ? (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES) : nullptr;
  const int bm = g.bm, nw = g.nw;
  const long total = g.tiles * g.splits;
  if (total > 0x7fffffffL) {
    set_error("q4_linear(gemm): grid too large");
    return Q4_ERR_UNSUPPORTED;
  }
  const size_t smem = 2 * (size_t)bm * kAUnitsPerRow * 16;
  dim3 grid((unsigned)total);
  const int gs = w->groupsize;
  if (dtype == Q4_DTYPE_F16) {
    if (bm == 256) launch_tile<Q4_DTYPE_F16, 256, 2>(gp, gs, grid, smem, stream);
    else if (nw == 2) launch_tile<Q4_DTYPE_F16, 128, 2>(gp, gs, grid, smem, stream);
    else launch_tile<Q4_DTYPE_F16, 128, 1>(gp, gs, grid, smem, stream);
  } else {
    if (bm == 256) launch_tile<Q4_DTYPE_BF16, 256, 2>(gp, gs, grid, smem, stream);
    else if (nw == 2) launch_tile<Q4_DTYPE_BF16, 128, 2>(gp, gs, grid, smem, stream);
    else launch_tile<Q4_DTYPE_BF16, 128, 1>(gp, gs, grid, smem, stream);
  }
  if (g.splits > 1) launch_gemm_reduce(gp.partials, bias, y, M, w->N, g.splits, dtype, stream);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemm): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
