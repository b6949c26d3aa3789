// Prefill path for the layouts whose packed words cannot feed the MFMA directly:
// y[M, N] = x @ dequant(W) for AWQ and for GPTQ with g_idx (act-order), gfx950.
//
// An AWQ word holds 8 interleaved columns of ONE K row; an act-order GPTQ word holds 8 K
// rows that each belong to a different group.  In both cases the weight tile is unpacked
// cooperatively into LDS (the classic dequantize-to-LDS stage) and both MFMA operands are
// read from there:
//   * workgroup = 4 waves in a 2 x 2 arrangement, tile 128 x 128, K tile 64; each wave owns
//     a 64 x 64 block = 2 x 2 MFMA tiles of v_mfma_f32_32x32x16 (64 accumulator VGPRs),
//     so two or three workgroups share a CU and cover each other's barriers;
//   * producer: thread t < 128 owns an 8-row x 1-word patch (8 rows of one K block, 8
//     columns).  One byte permute per row pair and byte puts the same nibble positions of
//     two rows side by side, the mantissa splice turns them into halves, zero points are
//     subtracted exactly and each weight is multiplied once by its fp16 scale (the
//     reference's rounding).  The patch becomes eight 16-byte units (one per column,
//     8 consecutive K values each) written to LDS at [K block][column];
//   * act-order producer: every thread owns 4 packed words (8 K rows x 1 column each).  The
//     groups of the 8 rows are wave-uniform (g_idx[k]); scale and zero point of each row
//     are gathered from the checkpoint tensors (coalesced across the 64 columns of a wave,
//     L2 resident) and applied per weight -- no row of qweight is ever moved;
//   * LDS layouts: activations [row][K block] with the row stride padded to 9 units,
//     weights [K block][column]; both give conflict-free 128-bit fragment reads;
//   * double-buffered LDS, global loads for tile k+2 in flight while tile k is multiplied.
#include "q4_common.cuh"

namespace q4 {

constexpr int kABM = 128;  // rows per workgroup
constexpr int kABN = 128;  // columns per workgroup
constexpr int kABK = 64;   // K rows per tile
constexpr int kAUnits = kABK / 8 + 1;  // padded units per activation row

struct AwqGemmParams {
  // split-K as in the GPTQ GEMM: `splits` workgroups per output tile, fp32 partial tiles in
  // partials[split][M][N], combined by gemm_reduce_kernel
  float* __restrict__ partials;
  int splits;
  Problem p;
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

typedef __bf16 awq_bf16x2_t __attribute__((ext_vector_type(2)));
typedef float awq_float2_t __attribute__((ext_vector_type(2)));

// ACT = false: AWQ layout.  ACT = true: GPTQ layout with g_idx.
template <int DTYPE, bool ACT>
__global__ __launch_bounds__(256, 2) void gemm_awq_kernel(AwqGemmParams gp) {
  constexpr int A_TILE = kABM * kAUnits * 16;   // bytes
  constexpr int B_TILE = (kABK / 8) * kABN * 16;
  constexpr int A_LOADS = kABM * (kABK / 8) / 256;  // 16-byte activation loads per thread
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
  const int tiles_m = (M + kABM - 1) / kABM;
  const int tiles_all = tiles_m * (N / kABN);
  const int split = blockIdx.x / tiles_all;
  const int tile_id = blockIdx.x - split * tiles_all;
  const int tm = tile_id % tiles_m;
  const int tn = tile_id / tiles_m;
  const int m0 = tm * kABM;
  const int n0 = tn * kABN;
  const int KT_all = K / kABK;
  const int kt_begin = (int)((long)split * KT_all / gp.splits);  // this workgroup's K tiles
  const int KT = (int)((long)(split + 1) * KT_all / gp.splits);
  const int last_tile = KT - 1;
  const AwqSplice splice = awq_splice_consts();

  // ---- producer state
  // AWQ: threads 0..127 own K block pb (8 rows) x word pc (8 columns).
  // act-order: every thread owns column pn and K blocks pkb0, pkb0 + 2, pkb0 + 4, pkb0 + 6.
  const bool producer = ACT || tid < 128;
  const int pb = (tid >> 4) & 7;
  const int pc = tid & 15;
  const int pn = tid & 127;
  const int pkb0 = __builtin_amdgcn_readfirstlane(tid >> 7);  // wave-uniform
  const uint32_t* wsrc = ACT ? p.qweight + (size_t)pkb0 * N + n0 + pn
                             : p.qweight + (size_t)(pb * 8) * NC + (n0 >> 3) + pc;
  uint32_t braw[8];  // AWQ: 8 rows of one word column; act-order: 4 words (K blocks)
  uint4_t sraw;      // AWQ: 8 fp16 scales of the word's columns
  uint32_t zraw;     // AWQ: 8 zero-point nibbles
  auto load_b = [&](int kt) {
    if constexpr (ACT) {
#pragma unroll
      for (int i = 0; i < 4; ++i) braw[i] = wsrc[(size_t)(kt * (kABK / 8) + 2 * i) * N];
    } else if (producer) {
#pragma unroll
      for (int r = 0; r < 8; ++r) braw[r] = wsrc[(size_t)(kt * kABK + r) * NC];
      const int g = min((kt * kABK + pb * 8) / p.groupsize, p.num_groups - 1);
      sraw = *(const uint4_t*)(p.scales + (size_t)g * N + n0 + pc * 8);
      zraw = p.qzeros[(size_t)g * NC + (n0 >> 3) + pc];
    }
  };
  auto store_b_act = [&](int buf, int kt) {
    unsigned char* base = smem + 2 * A_TILE + buf * B_TILE;
    const int n = n0 + pn;
    const int zshift = (n & 7) * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kb = pkb0 + 2 * i;
      const int k0 = kt * kABK + kb * 8;
      // scale and -(1024 + zero) of the 8 rows of this word: groups are wave-uniform
      uint32_t sc[8], cz[8];
#pragma unroll
      for (int r = 0; r < 8; ++r) {
        int g = p.g_idx[k0 + r];
        g = min(max(g, 0), p.num_groups - 1);
        sc[r] = *(const uint16_t*)(p.scales + (size_t)g * N + n);
        const uint32_t z = (gptq_zero_plus_one(p.qzeros[(size_t)g * NC + (n >> 3)]) >> zshift) & 0xFu;
        cz[r] = 0xE400u | z;
      }
      const uint32_t w = braw[i];
      uint32_t o[4];
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) {
        // rows pr and pr + 4 share one splice (nibbles 16 bits apart)
        const uint32_t q2 = ((w >> (4 * pr)) & splice.mask_lo) | splice.magic;
        const half2_t dq = as_half2(q2) + as_half2(cz[pr] | (cz[pr + 4] << 16));  // exact q - z
        if constexpr (DTYPE == Q4_DTYPE_F16) {
          o[pr] = as_u32(dq * as_half2(sc[pr] | (sc[pr + 4] << 16)));  // one fp16 rounding
        } else {
          const half2_t s2 = as_half2(sc[pr] | (sc[pr + 4] << 16));
          const awq_float2_t f = {(float)dq.x * (float)s2.x, (float)dq.y * (float)s2.y};
          o[pr] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, awq_bf16x2_t));
        }
      }
      // o holds rows (0,4),(1,5),(2,6),(3,7): back to natural K order for the unit
      uint4_t unit;
      unit.x = (o[0] & 0xFFFFu) | (o[1] << 16);
      unit.y = (o[2] & 0xFFFFu) | (o[3] << 16);
      unit.z = (o[0] >> 16) | (o[1] & 0xFFFF0000u);
      unit.w = (o[2] >> 16) | (o[3] & 0xFFFF0000u);
      *(uint4_t*)(base + ((size_t)kb * kABN + pn) * 16) = unit;
    }
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
      *(uint4_t*)(base + ((size_t)pb * kABN + pc * 8 + col) * 16) = unit;
    }
  };

  auto store_b = [&](int buf, int kt) {
    if constexpr (ACT) store_b_act(buf, kt);
    else store_b_awq(buf);
  };

  // ---- activation tile: global -> registers -> LDS (natural K order)
  const uint16_t* xs = (const uint16_t*)p.x;
  uint4_t areg[A_LOADS];
  auto load_a = [&](int kt) {
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + 256 * i;
      const int m = u >> 3, kb = u & 7;
      const int row = min(m0 + m, M - 1);  // rows past M re-read the last row, never stored
      areg[i] = *(const uint4_t*)(xs + (size_t)row * K + kt * kABK + kb * 8);
    }
  };
  auto store_a = [&](int buf) {
    unsigned char* base = smem + buf * A_TILE;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
      const int u = tid + 256 * i;
      const int m = u >> 3, kb = u & 7;
      *(uint4_t*)(base + (m * kAUnits + kb) * 16) = areg[i];
    }
  };

  float16_t acc[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a)
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[a][b][r] = 0.f;

  load_a(kt_begin);
  load_b(kt_begin);
  store_a(0);
  store_b(0, kt_begin);
  load_a(min(kt_begin + 1, last_tile));
  load_b(min(kt_begin + 1, last_tile));
  __syncthreads();

  const int a_off = ((wm * 64 + j) * kAUnits + kq) * 16;
  const int b_off = (kq * kABN + wn * 64 + j) * 16;

  for (int kt = kt_begin; kt < KT; ++kt) {
    const int cur = (kt - kt_begin) & 1;
    // the other buffer was last read in tile kt-1, before the barrier that ended it
    store_a(cur ^ 1);
    store_b(cur ^ 1, min(kt + 1, last_tile));
    const int kt2 = min(kt + 2, last_tile);
    load_a(kt2);
    load_b(kt2);
    const unsigned char* ab = smem + cur * A_TILE + a_off;
    const unsigned char* bb = smem + 2 * A_TILE + cur * B_TILE + b_off;
#pragma unroll
    for (int s = 0; s < kABK / 16; ++s) {
      uint4_t af[2], bf[2];
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) af[mt] = *(const uint4_t*)(ab + (mt * 32 * kAUnits + 2 * s) * 16);
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) bf[nt] = *(const uint4_t*)(bb + ((2 * s) * kABN + nt * 32) * 16);
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
          if constexpr (DTYPE == Q4_DTYPE_F16) {
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                __builtin_bit_cast(half8_t, af[mt]), __builtin_bit_cast(half8_t, bf[nt]), acc[mt][nt], 0, 0, 0);
          } else {
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(bf16x8_t, af[mt]), __builtin_bit_cast(bf16x8_t, bf[nt]), acc[mt][nt], 0, 0, 0);
          }
        }
    }
    __syncthreads();
  }

  // ---- epilogue: register r of lane (j, kq) is row 8*(r/4) + 4*kq + r%4, column j
  if (gp.splits > 1) {
    float* part = gp.partials + (size_t)split * M * N;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const int n = n0 + wn * 64 + nt * 32 + j;
#pragma unroll
      for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int m = m0 + wm * 64 + mt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
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
    for (int mt = 0; mt < 2; ++mt) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + mt * 32 + 8 * (r >> 2) + 4 * kq + (r & 3);
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

// 128 x 128 tiles, ~1.0 us per K tile alone on a CU, ~1.9 us when two workgroups share it
int gemm_awq_splits(int M, int K, int N) {
  if (K % q4::kABK != 0 || N % q4::kABN != 0) return 1;
  const long tiles = (long)((M + q4::kABM - 1) / q4::kABM) * (N / q4::kABN);
  return tiles < 256 ? gemm_pick_splits(tiles, K / q4::kABK, M, N, 1.0, 1.9) : 1;
}

int launch_gemm_awq(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                    void* workspace, size_t workspace_bytes, hipStream_t stream) {
  using namespace q4;
  if (!gemm_awq_supported(w, M, dtype)) {
    set_error("q4_linear(gemm/awq): unsupported problem (M=%d K=%d N=%d groupsize=%d)", M, w->K, w->N,
              w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  AwqGemmParams gp;
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, w->g_idx, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  int splits = gemm_awq_splits(M, w->K, w->N);
  if (splits > 1 && (workspace == nullptr ||
                     workspace_bytes < Q4_WORKSPACE_COUNTER_BYTES + (size_t)splits * M * w->N * sizeof(float)))
    splits = 1;  // no room for partial tiles: one workgroup per whole tile
  gp.splits = splits;
  gp.partials = splits > 1 ? (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES) : nullptr;
  const long total = (long)((M + kABM - 1) / kABM) * (w->N / kABN) * splits;
  if (total > 0x7fffffffL) {
    set_error("q4_linear(gemm/awq): grid too large");
    return Q4_ERR_UNSUPPORTED;
  }
  const size_t smem = 2 * (size_t)kABM * kAUnits * 16 + 2 * (size_t)(kABK / 8) * kABN * 16;
  const bool act = w->layout == Q4_LAYOUT_GPTQ;
  auto launch = [&](auto k) {
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
    hipLaunchKernelGGL(k, dim3((unsigned)total), dim3(256), smem, stream, gp);
  };
  if (dtype == Q4_DTYPE_F16) {
    if (act) launch(gemm_awq_kernel<Q4_DTYPE_F16, true>);
    else launch(gemm_awq_kernel<Q4_DTYPE_F16, false>);
  } else {
    if (act) launch(gemm_awq_kernel<Q4_DTYPE_BF16, true>);
    else launch(gemm_awq_kernel<Q4_DTYPE_BF16, false>);
  }
  if (splits > 1) launch_gemm_reduce(gp.partials, bias, y, M, w->N, splits, dtype, stream);
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemm/awq): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
