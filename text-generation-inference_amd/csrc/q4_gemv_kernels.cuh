// Decode kernels (device code shared by the translation units that instantiate them).
//
// Decode path: y[M, N] = x @ dequant(W) for small M (16 rows per workgroup row-chunk).
//
// HBM-bound: the packed weights are read exactly once with wide loads and never written
// back.  All three kernels share one structure (wave64):
//   * the B operand of a 16x16x32 MFMA wants, per lane, 8 consecutive K values of one
//     column (column = lane % 16, K block = lane / 16).  The matrix core then performs both
//     the multiply and the reduction across the four K blocks of the wave; the VALU only
//     unpacks nibbles (about one operation per weight);
//   * nibbles become halves by splicing them into the mantissa of 1024.0 (q4_common.cuh),
//     zero points are subtracted exactly in fp16 and, when groups are contiguous in K, the
//     group scale is factored out of the K sum and applied to the fp32 group accumulator;
//   * the activation slab of the workgroup is staged once in LDS in the K order the unpack
//     produces, so no weight is ever repacked;
//   * split-K: `wk` waves of a workgroup take consecutive K ranges and are combined through
//     LDS in fixed order; `splits` workgroups write fp32 partials to the workspace and the
//     last one to arrive (ticket counter) adds them in split order and writes the output.
//     The result is deterministic and needs no memset: the last workgroup resets its ticket.
//
// gemv_gptq_kernel      GPTQ layout, groups contiguous in K.  A packed word *is* one lane's
//                       B operand; a lane loads 4 adjacent columns x 1 packed row with one
//                       128-bit load (256-byte row segments per 16 lanes), word t feeds
//                       MFMA t.
// gemv_gptq_act_kernel  GPTQ layout with g_idx (act-order): every K row has its own group.
//                       Scales and zero points of the workgroup's columns sit in an LDS
//                       table indexed by g_idx[k]; they are applied per weight.
// gemv_awq_kernel       AWQ layout: a word holds 8 interleaved columns of one K row.  A lane
//                       loads an 8-row x 2-word patch and transposes nibbles in registers
//                       (one byte permute per row pair and byte) into 16 B operands.
//
// Workgroup ids are laid out split-major so that all splits of a column tile land on the
// same XCD (id % 8) and the partials stay in that XCD's L2.
#pragma once
#include <type_traits>

#include "q4_common.cuh"

namespace q4 {

constexpr int kChunkSteps = 4;                // 32-row MFMA steps per software-pipelined chunk
constexpr int kChunkRows = 32 * kChunkSteps;  // 128 K rows
constexpr int kPrefetch = 2;                  // chunks of weight loads in flight per wave
constexpr int kRowsPerBlock = 16;             // activation rows per workgroup (MFMA M)

struct GemvParams {
  Problem p;
  float* __restrict__ partials;
  uint32_t* __restrict__ tickets;
  int wcol, wk, splits;
  unsigned long long* __restrict__ cells;  // fixed-point accumulation cells [M][N] (workspace)
  int fixed_point_split;  // fp16 outputs: combine the splits with one 64-bit atomic per element
  int slab_stride;  // bytes between activation rows in LDS
  int slab_bytes;   // size of the activation slab region
  int kr_max;        // largest K range of a workgroup (K is dealt out in 128-row chunks)
  int partial_rows;  // rows of one split's slice of `partials` (M; grouped launches: all pairs)
  int rows_per_block;  // activation rows per workgroup: 16, or 32 (two MFMA row blocks per unpacked word)
  MoeView moe;       // grouped launches only (MOE kernels): blockIdx.z is the expert
  // How the K / 128 chunks are dealt out (set_k_deal): workgroup `split` takes kd_Q chunks, the
  // first kd_R workgroups one more; inside a workgroup of kd_Q (+1) chunks wave wkk takes
  // kd_q0 (kd_q1) chunks, the first kd_r0 (kd_r1) waves one more.  No division on the device.
  int ntiles, kd_Q, kd_R, kd_q0, kd_r0, kd_q1, kd_r1;
  int rows_per_block_alloc;  // lean kernel: activation rows every wave's piece of LDS has room for
  int wave_slab;             // lean kernel: 1 = every wave stages its own K range, 0 = one slab per workgroup
#ifdef Q4_PHASE_STAMPS
  unsigned long long* __restrict__ stamps;  // [workgroups][waves][8] clock readings, or nullptr
#endif
};

// Fills the K partition of gp for `chunks` chunks over `splits` workgroups of `wk` waves
// (splits * wk <= chunks) and returns the largest K range of a workgroup in rows.
inline int set_k_deal(GemvParams& gp, int chunks, int splits, int wk) {
  gp.kd_Q = chunks / splits;
  gp.kd_R = chunks % splits;
  gp.kd_q0 = gp.kd_Q / wk;
  gp.kd_r0 = gp.kd_Q % wk;
  gp.kd_q1 = (gp.kd_Q + 1) / wk;
  gp.kd_r1 = (gp.kd_Q + 1) % wk;
  return (gp.kd_Q + (gp.kd_R > 0 ? 1 : 0)) * 128;
}
// Largest K range of a wave under the same partition, in rows.
inline int max_wave_rows(const GemvParams& gp) {
  const int a = gp.kd_q0 + (gp.kd_r0 > 0 ? 1 : 0), b = gp.kd_R > 0 ? gp.kd_q1 + (gp.kd_r1 > 0 ? 1 : 0) : 0;
  return (a > b ? a : b) * 128;
}

// Buffer loads: a scalar descriptor (base, byte count), one 32-bit lane offset and a scalar offset
// that moves.  A lane offset at or past the byte count makes the load return zeros without a
// memory access, which is how the decode loops keep their refill loads free of branches: with a
// branch around a load the compiler cannot count the loads in flight and waits for all of them.
typedef __amdgpu_buffer_rsrc_t direct_rsrc_t;
__device__ __forceinline__ direct_rsrc_t direct_rsrc(const void* base, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ uint32_t scalar_u32(uint32_t v) { return __builtin_amdgcn_readfirstlane(v); }

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

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float float2_t __attribute__((ext_vector_type(2)));

// half2 of exact small integers -> packed bf16 pair (exact; v_cvt_pk_bf16_f32).
__device__ __forceinline__ uint32_t pack_bf16_pair(half2_t h) {
  const float2_t f = {(float)h.x, (float)h.y};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
}

// One 16x16x32 MFMA; `b` holds eight weights as four half2.
template <int DTYPE>
__device__ __forceinline__ float4_t mfma16(const uint4_t a, const half2_t b[4], float4_t c) {
  if constexpr (DTYPE == Q4_DTYPE_F16) {
    uint4_t bu;
    bu.x = as_u32(b[0]); bu.y = as_u32(b[1]); bu.z = as_u32(b[2]); bu.w = as_u32(b[3]);
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a),
                                                  __builtin_bit_cast(half8_t, bu), c, 0, 0, 0);
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

// ---------------------------------------------------------------------------------------
// Work decomposition shared by the kernels.
struct Decomp {
  int tid, lane, wave, wc, wkk, j, kq, nthreads;
  int tile_cols, ntiles, tile, split;
  int KR, KW, kwg0, kw0;  // K range of the workgroup [kwg0, kwg0 + KR) and of the wave [kw0, kw0 + KW)
  int kwo;                // kw0 - kwg0: the wave's offset inside the workgroup's slab
  int mb, mloc;  // first activation row of this workgroup and number of live rows (<= 16)
};

__device__ __forceinline__ Decomp make_decomp(const GemvParams& gp, int wave_cols) {
  Decomp d;
  d.tid = threadIdx.x;
  d.lane = d.tid & 63;
  d.wave = __builtin_amdgcn_readfirstlane(d.tid >> 6);  // wave-uniform: keeps index math scalar
  d.wc = d.wave % gp.wcol;
  d.wkk = d.wave / gp.wcol;
  d.j = d.lane & 15;
  d.kq = d.lane >> 4;
  d.nthreads = blockDim.x;
  d.tile_cols = wave_cols * gp.wcol;
  d.ntiles = gp.ntiles;
  d.tile = blockIdx.x % (unsigned)d.ntiles;
  d.split = blockIdx.x / (unsigned)d.ntiles;
  // K is dealt out in chunks of 128 rows, first over the `splits` workgroups, then over the wk
  // waves of each, as evenly as the counts allow (ranges differ by at most one chunk)
  const bool big = d.split < gp.kd_R;
  const int g0 = d.split * gp.kd_Q + min(d.split, gp.kd_R);
  const int wq = big ? gp.kd_q1 : gp.kd_q0, wr = big ? gp.kd_r1 : gp.kd_r0;
  d.kwg0 = g0 * kChunkRows;
  d.KR = (gp.kd_Q + (big ? 1 : 0)) * kChunkRows;
  d.kw0 = (g0 + d.wkk * wq + min(d.wkk, wr)) * kChunkRows;
  d.KW = (wq + (d.wkk < wr ? 1 : 0)) * kChunkRows;
  d.kwo = d.kw0 - d.kwg0;
  d.mb = blockIdx.y * gp.rows_per_block;
  d.mloc = min(gp.rows_per_block, gp.p.M - d.mb);
  return d;
}

// Clock readings of a wave at the phase boundaries of a decode launch.  Measurement builds only
// (-DQ4_PHASE_STAMPS, a second library next to the product one): the readings stay in scalar
// registers and go to memory with one store per wave right before it ends, so nothing is added
// to the path being timed except the reads of the constant 100 MHz counter themselves.  In the
// product build every member is empty and the calls compile to nothing.
//   0 entry   1 activations staged (behind the workgroup barrier, where there is one)
//   2 first chunk consumed   3 last chunk consumed (K loop done)   4 K waves of the workgroup
//   combined through LDS   5 split-K combine returned (atomic / ticket)   6 first weight loads
//   issued   7 exit
struct PhaseStamps {
#ifdef Q4_PHASE_STAMPS
  unsigned long long t[8];
  __device__ __forceinline__ PhaseStamps() {
#pragma unroll
    for (int i = 0; i < 8; ++i) t[i] = 0ull;
    t[0] = __builtin_amdgcn_s_memrealtime();
  }
  __device__ __forceinline__ void mark(int i) { t[i] = __builtin_amdgcn_s_memrealtime(); }
  // reading taken once `v` has been computed (pins the stamp behind the work that makes v)
  __device__ __forceinline__ void mark_after(int i, float v) {
    asm volatile("" ::"v"(v));
    mark(i);
  }
  // all eight readings of this wave -> base[workgroup][wave][8]
  __device__ __forceinline__ void flush_to(unsigned long long* base, int lane, int wave) {
    if (base == nullptr) return;
    mark(7);
    if (lane == 0) {
      unsigned long long* dst = base + (((size_t)blockIdx.y * gridDim.x + blockIdx.x) * (blockDim.x >> 6) + wave) * 8;
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i] = t[i];
    }
  }
  __device__ __forceinline__ void flush(const GemvParams& gp, const Decomp& d) { flush_to(gp.stamps, d.lane, d.wave); }
#else
  __device__ __forceinline__ void mark(int) {}
  __device__ __forceinline__ void mark_after(int, float) {}
  __device__ __forceinline__ void flush(const GemvParams&, const Decomp&) {}
#endif
};

// Entry of a grouped (MOE) decode launch: narrows gp to the expert blockIdx.z.  Returns false
// when this workgroup's row block lies beyond the expert's rows (the whole workgroup leaves).
// `rows` receives the activation-row map of the block, or nullptr when x is in sorted order.
__device__ __forceinline__ bool moe_enter_decode(GemvParams& gp, const int32_t*& rows, bool half_width_output = false) {
  const int row0 = moe_enter(gp.p, gp.moe, blockIdx.z);
  // the gated-MLP epilogue writes N / 2 columns per row
  if (half_width_output) gp.p.y = (uint16_t*)gp.p.y - (size_t)row0 * (gp.p.N >> 1);
  if (gp.p.M <= (int)blockIdx.y * gp.rows_per_block) return false;
  gp.partials += (size_t)row0 * gp.p.N;
  rows = gp.moe.x_rows != nullptr ? gp.moe.x_rows + row0 + blockIdx.y * gp.rows_per_block : nullptr;
  return true;
}

// Activation slab [mloc][KR] -> LDS.  The global loads are issued before the weight loads
// (memory returns in issue order, so L2 hits must not queue behind the HBM stream they are
// needed to consume) and stored after them.  PERMUTE stores every 8-block in the K order
// [0,4,1,5,2,6,3,7] of the GPTQ nibble splice.
template <bool PERMUTE, int LOADS = 2>
struct SlabStager {
  static constexpr int kLoads = LOADS;  // 16-byte activation loads per thread in flight before the weight loads
  static constexpr int kBatch = 4;      // ... and per round of what is left (many rows, a long K range)
  uint4_t xv[kLoads];
  const uint16_t* xs;
  const int32_t* rows;  // grouped launches: row of x behind every staged row, else nullptr
  const int32_t* cols;  // column of x behind every K row of the workgroup's range, else nullptr
  // Item i of a thread is 16-byte block tid + i * nthreads of the slab, counted row by row.  Its
  // (row, block) is walked incrementally: one division per thread, none per item.
  int kb_per_row, mloc;
  int m0, kb0;   // the thread's first item
  int dm, dkb;   // (row, block) step between a thread's items: nthreads = dm * kb_per_row + dkb

  __device__ __forceinline__ void advance(int& m, int& kb) const {
    m += dm;
    kb += dkb;
    if (kb >= kb_per_row) {
      kb -= kb_per_row;
      ++m;
    }
  }
  __device__ __forceinline__ uint4_t fetch(const GemvParams& gp, int m, int kb) const {
    const int mr = rows != nullptr ? rows[m] : m;
    if (cols != nullptr) {
      // eight scattered columns of the row (it stays in L2); a bad index is clamped
      const uint16_t* row = xs + (size_t)mr * gp.p.K;
      const uint4_t p0 = *(const uint4_t*)(cols + kb * 8);
      const uint4_t p1 = *(const uint4_t*)(cols + kb * 8 + 4);
      const int last = gp.p.K - 1;
      auto at = [&](uint32_t i) { return (uint32_t)row[min(max((int)i, 0), last)]; };
      uint4_t o;
      o.x = at(p0.x) | (at(p0.y) << 16);
      o.y = at(p0.z) | (at(p0.w) << 16);
      o.z = at(p1.x) | (at(p1.y) << 16);
      o.w = at(p1.z) | (at(p1.w) << 16);
      return o;
    }
    return *(const uint4_t*)(xs + (size_t)mr * gp.p.K + kb * 8);
  }
  __device__ __forceinline__ void issue(const GemvParams& gp, const Decomp& d, const int32_t* row_map = nullptr) {
    rows = row_map;
    cols = gp.p.x_perm != nullptr ? gp.p.x_perm + d.kwg0 : nullptr;
    xs = (const uint16_t*)gp.p.x + (row_map != nullptr ? 0 : (size_t)d.mb * gp.p.K) + (cols != nullptr ? 0 : d.kwg0);
    kb_per_row = d.KR >> 3;
    mloc = d.mloc;
    m0 = d.tid / kb_per_row;
    kb0 = d.tid - m0 * kb_per_row;
    dm = d.nthreads / kb_per_row;
    dkb = d.nthreads - dm * kb_per_row;
    int m = m0, kb = kb0;
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      if (m < mloc) xv[u] = fetch(gp, m, kb);
      advance(m, kb);
    }
  }
  __device__ __forceinline__ void put(const GemvParams& gp, unsigned char* smem, int m, int kb, uint4_t v) const {
    uint4_t o = v;
    if constexpr (PERMUTE) {
      o.x = (v.x & 0xFFFFu) | (v.z << 16);
      o.y = (v.x >> 16) | (v.z & 0xFFFF0000u);
      o.z = (v.y & 0xFFFFu) | (v.w << 16);
      o.w = (v.y >> 16) | (v.w & 0xFFFF0000u);
    }
    *(uint4_t*)(smem + (size_t)m * gp.slab_stride + kb * 16) = o;
  }
  __device__ __forceinline__ void store(const GemvParams& gp, const Decomp& d, unsigned char* smem) {
    (void)d;
    int m = m0, kb = kb0;
#pragma unroll
    for (int u = 0; u < kLoads; ++u) {
      if (m < mloc) put(gp, smem, m, kb, xv[u]);
      advance(m, kb);
    }
    // the rest in rounds of kBatch loads per thread: one memory round trip per round, not per
    // load (a row past the end is clamped for the load and not stored)
    while (m < mloc) {
      uint4_t t[kBatch];
      int ms[kBatch], kbs[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; ++u) {
        ms[u] = m;
        kbs[u] = kb;
        t[u] = fetch(gp, min(m, mloc - 1), kb);
        advance(m, kb);
      }
#pragma unroll
      for (int u = 0; u < kBatch; ++u)
        if (ms[u] < mloc) put(gp, smem, ms[u], kbs[u], t[u]);
    }
  }
};

// Row (relative to the workgroup's first) of accumulator slot r of a lane: an MFMA row block
// gives a lane rows 4*kq .. 4*kq + 3; slots 4..7 are the second block of 16 rows.
// KQROWS (the AWQ kernel, whose MFMA rows are (activation row, column) pairs): lane block kq
// holds rows kq, kq + 4, ..
template <bool KQROWS = false>
__device__ __forceinline__ int out_row(const Decomp& d, int r) {
  if constexpr (KQROWS) return d.kq + 4 * r;
  return 4 * d.kq + (r & 3) + ((r >> 2) << 4);
}

// 64-bit accumulation cell of the fixed-point split-K combine (up to 14 splits):
//   bits 60..63  arrivals
//   bits 55..58  arrivals whose partial sum was -inf or NaN
//   bits 51..54  arrivals whose partial sum was +inf or NaN
//   bits  0..50  sum of the finite partial sums, 28 fractional bits, two's complement running
//                into the fields above (read back with a bias of 2^50)
// A partial sum beyond +-2^17 (twice the largest fp16) counts as an infinity of its sign, so 14
// finite ones stay below 2^49.  The combined value is NaN when both non-finite fields are set
// (a NaN partial, or +inf meeting -inf), else +-inf when one is, else the fixed-point sum: what
// fp32 addition of the partials gives in any order, as long as no partial leaves +-2^17 (one
// that does makes the fp16 output infinite or, when such partials cancel, NaN).
__device__ __forceinline__ unsigned long long cell_increment(float v) {
  constexpr unsigned long long kArrival = 1ull << 60, kPos = 1ull << 51, kNeg = 1ull << 55;
  if (fabsf(v) <= 131072.f) return kArrival + (unsigned long long)__float2ll_rn(v * 268435456.f);
  return kArrival + (v < 0.f ? 0ull : kPos) + (v > 0.f ? 0ull : kNeg);  // NaN compares false both ways
}
__device__ __forceinline__ bool cell_complete(unsigned long long now, int splits) {
  return (int)((now + (1ull << 50)) >> 60) == splits;
}
__device__ __forceinline__ float cell_value(unsigned long long now) {
  const unsigned long long t = now + (1ull << 50);
  const bool pos = ((t >> 51) & 15ull) != 0, neg = ((t >> 55) & 15ull) != 0;
  const float f = (float)((long long)(t & ((1ull << 51) - 1)) - (1ll << 50)) * (1.0f / 268435456.f);
  if (pos || neg) return pos && neg ? __builtin_nanf("") : (pos ? __builtin_inff() : -__builtin_inff());
  return f;
}

// Everything after the K loop.  out[t][r] is the fp32 sum of output row out_row(r) (relative
// to the workgroup's first row) and column col0 + t: every lane owns NT adjacent columns.
// FUSE (NT = 8): gated-MLP epilogue.  out[0..3] are four gate columns col0 .. col0 + 3 and
// out[4..7] the matching up columns N/2 + col0 ..; the output is act(gate) * up, [M, N/2].
template <int DTYPE, int NT, int RMAX, bool FUSE = false, bool KQROWS = false>
__device__ __forceinline__ void gemv_finish_impl(const GemvParams& gp, const Decomp& d,
                                                 float (&out)[NT][RMAX], int col0,
                                                 unsigned char* smem, PhaseStamps& ps) {
  const Problem& p = gp.p;
  const int N = p.N;
  // ---- combine the wk waves of the workgroup through LDS (fixed order)
  if (gp.wk > 1) {
    __syncthreads();  // everyone is done with the slab / tables
    float* red = (float*)smem;
    if (d.wkk > 0) {
      float* dst = red + ((size_t)((d.wkk - 1) * gp.wcol + d.wc) * NT * RMAX) * 64 + d.lane;
#pragma unroll
      for (int t = 0; t < NT; ++t)
#pragma unroll
        for (int r = 0; r < RMAX; ++r) dst[(t * RMAX + r) * 64] = out[t][r];
    }
    __syncthreads();
    if (d.wkk == 0) {
      for (int w = 1; w < gp.wk; ++w) {
        const float* src = red + ((size_t)((w - 1) * gp.wcol + d.wc) * NT * RMAX) * 64 + d.lane;
#pragma unroll
        for (int t = 0; t < NT; ++t)
#pragma unroll
          for (int r = 0; r < RMAX; ++r) out[t][r] += src[(t * RMAX + r) * 64];
      }
    }
  }
  ps.mark_after(4, out[0][0]);

  uint16_t* y = (uint16_t*)p.y;
  const int half_n = N >> 1;
  if constexpr (FUSE) {
    if (gp.splits == 1) {
      if (d.wkk == 0) {
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
          const int m = out_row<KQROWS>(d, r);
          if (m < d.mloc) {
            uint32_t o[NT / 2];
#pragma unroll
            for (int t = 0; t < NT / 2; ++t) {
              const uint16_t g = finish_output<DTYPE>(out[t][r], p.bias, col0 + t);
              const uint16_t u = finish_output<DTYPE>(out[NT / 2 + t][r], p.bias, half_n + col0 + t);
              o[t] = act_mul<DTYPE>(g, u, p.gate_up_act - 1);
            }
            uint2_t packed;
            packed.x = o[0] | (o[1] << 16);
            packed.y = o[2] | (o[3] << 16);
            *(uint2_t*)(y + (size_t)(d.mb + m) * half_n + col0) = packed;
          }
        }
      }
      return;
    }
  }
  if (gp.splits == 1) {
    if (d.wkk == 0) {
#pragma unroll
      for (int r = 0; r < RMAX; ++r) {
        const int m = out_row<KQROWS>(d, r);
        if (m < d.mloc) {
          uint16_t* dst = y + (size_t)(d.mb + m) * N + col0;
          uint16_t o[NT];
#pragma unroll
          for (int t = 0; t < NT; ++t) o[t] = finish_output<DTYPE>(out[t][r], p.bias, col0 + t);
          if constexpr (NT == 1) {
            dst[0] = o[0];
          } else if constexpr (NT == 2) {
            *(uint32_t*)dst = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
          } else {
#pragma unroll
            for (int t = 0; t < NT; t += 4) {
              uint2_t packed;
              packed.x = (uint32_t)o[t] | ((uint32_t)o[t + 1] << 16);
              packed.y = (uint32_t)o[t + 2] | ((uint32_t)o[t + 3] << 16);
              *(uint2_t*)(dst + t) = packed;
            }
          }
        }
      }
    }
    return;
  }

  // ---- cross-workgroup split-K, fp16: one 64-bit atomic per output element and workgroup.
  // The cell of an element accumulates the partial sums in fixed point (integer addition: the
  // total does not depend on the arrival order) next to the number of arrivals (cell_increment
  // above).  The add returns the previous contents, so the workgroup that brings the count to
  // `splits` holds the complete sum, writes the output and clears the cell: one memory round
  // trip where partial store -> ticket -> re-read takes three.  The cells must be zero before
  // the first call; they are left zero.
  if constexpr (DTYPE == Q4_DTYPE_F16 && !FUSE) {
    if (gp.fixed_point_split) {
      if constexpr (NT >= 4) {
        // A row's sums sit in the 16 lanes of one K block, NT adjacent columns each: issued
        // from there, an atomic instruction touches 16 separate groups of cells (with the AWQ
        // kernel's 16 columns per lane: 16 cache lines).  The wave's sums go through LDS so that
        // a lane owns columns lane, lane + 64, .. of one row: every instruction then covers 64
        // consecutive cells with all lanes active.  The tiles sit behind the K-wave partials.
        constexpr int PER_LANE = NT >= 4 ? NT / 4 : 1;  // 16 * NT columns over 64 lanes
        constexpr int TW = 16 * NT;
        constexpr int TILE_ROWS = KQROWS ? (4 * RMAX < kRowsPerBlock ? 4 * RMAX : kRowsPerBlock) : (RMAX < 4 ? RMAX : kRowsPerBlock);
        if (gp.wk == 1 && gp.wcol > 1) __syncthreads();  // other column waves may still read the slab
        float* tile = (float*)smem + (size_t)(gp.wk - 1) * gp.wcol * NT * RMAX * 64 + (size_t)d.wc * TILE_ROWS * TW;
        if (d.wkk == 0) {
#pragma unroll
          for (int r = 0; r < RMAX; ++r) {
            const int m = out_row<KQROWS>(d, r);
            if (m < d.mloc) {
#pragma unroll
              for (int t = 0; t < NT; ++t) tile[m * TW + d.j * NT + t] = out[t][r];
            }
          }
        }
        // Several rows: they are dealt to the K waves of the column wave, every wave with the adds
        // of two rows in flight.  (One wave taking the rows in turn pays a memory round trip per
        // row; the adds of several rows issued by one wave made the splits of a row arrive together
        // and measured 5-20 % slower than that.)
        const bool deal = d.mloc > 1 && gp.wk > 1;
        if (deal) __syncthreads();  // the tile is visible to the other K waves
        if (deal || d.wkk == 0) {
          const int nbase = col0 - d.j * NT;  // first column of this wave
          const int step = deal ? gp.wk : 1;
          for (int m0 = deal ? d.wkk : 0; m0 < d.mloc; m0 += 2 * step) {
            const int m1 = m0 + step;
            const bool two = deal && m1 < d.mloc;
            unsigned long long* cell0 = gp.cells + (size_t)(d.mb + m0) * N + nbase + d.lane;
            unsigned long long* cell1 = gp.cells + (size_t)(d.mb + (two ? m1 : m0)) * N + nbase + d.lane;
            unsigned long long before0[PER_LANE], inc0[PER_LANE], before1[PER_LANE], inc1[PER_LANE];
#pragma unroll
            for (int u = 0; u < PER_LANE; ++u) {
              inc0[u] = cell_increment(tile[m0 * TW + d.lane + 64 * u]);
              before0[u] = __hip_atomic_fetch_add(cell0 + 64 * u, inc0[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (two) {
#pragma unroll
              for (int u = 0; u < PER_LANE; ++u) {
                inc1[u] = cell_increment(tile[m1 * TW + d.lane + 64 * u]);
                before1[u] = __hip_atomic_fetch_add(cell1 + 64 * u, inc1[u], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              }
            }
            ps.mark_after(5, __builtin_bit_cast(float, (uint32_t)before0[0]));
#pragma unroll
            for (int u = 0; u < PER_LANE; ++u) {
              const unsigned long long now = before0[u] + inc0[u];
              if (cell_complete(now, gp.splits)) {
                const int n = nbase + d.lane + 64 * u;
                y[(size_t)(d.mb + m0) * N + n] = finish_output<DTYPE>(cell_value(now), p.bias, n);
                __hip_atomic_store(cell0 + 64 * u, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              }
            }
            if (two) {
#pragma unroll
              for (int u = 0; u < PER_LANE; ++u) {
                const unsigned long long now = before1[u] + inc1[u];
                if (cell_complete(now, gp.splits)) {
                  const int n = nbase + d.lane + 64 * u;
                  y[(size_t)(d.mb + m1) * N + n] = finish_output<DTYPE>(cell_value(now), p.bias, n);
                  __hip_atomic_store(cell1 + 64 * u, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                }
              }
            }
          }
        }
        return;
      }
      if (d.wkk == 0) {
        unsigned long long* cells = gp.cells;
#pragma unroll
        for (int r = 0; r < RMAX; ++r) {
          const int m = out_row<KQROWS>(d, r);
          if (m < d.mloc) {
            unsigned long long* cell = cells + (size_t)(d.mb + m) * N + col0;
            unsigned long long before[NT], inc[NT];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              inc[t] = cell_increment(out[t][r]);
              before[t] = __hip_atomic_fetch_add(cell + t, inc[t], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
#pragma unroll
            for (int t = 0; t < NT; ++t) {
              const unsigned long long now = before[t] + inc[t];
              if (cell_complete(now, gp.splits)) {
                y[(size_t)(d.mb + m) * N + col0 + t] = finish_output<DTYPE>(cell_value(now), p.bias, col0 + t);
                __hip_atomic_store(cell + t, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
              }
            }
          }
        }
      }
      return;
    }
  }

  // ---- cross-workgroup split-K: write the partial, take a ticket, last one reduces.
  // Partials and the ticket move with agent-scope relaxed atomics (coherent loads/stores
  // that bypass the per-XCD L2 state) instead of release/acquire fences: a fence here
  // would write back and invalidate the whole L2 once per workgroup, which costs more
  // than the kernel itself.  Ordering comes from waiting for the stores to be
  // acknowledged (vmcnt(0)) before the workgroup barrier that precedes the ticket.
  if (d.wkk == 0) {
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      const int m = out_row<KQROWS>(d, r);
      if (m < d.mloc) {
        float* dst = gp.partials + ((size_t)d.split * gp.partial_rows + d.mb + m) * N + col0;
#pragma unroll
        for (int t = 0; t < NT; ++t)
          __hip_atomic_store(dst + (FUSE && t >= NT / 2 ? half_n + t - NT / 2 : t), out[t][r], __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  __shared__ uint32_t ticket_s;
  uint32_t* ticket = gp.tickets + (blockIdx.z * gridDim.y + blockIdx.y) * d.ntiles + d.tile;
  if (d.tid == 0) {
    ticket_s = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  ps.mark(5);
  if (ticket_s != (uint32_t)(gp.splits - 1)) return;
  {
    const size_t sstride = (size_t)gp.partial_rows * N;
    // sum of the partials of one output element, in split order
    auto total = [&](int m, int n) {
      const float* src = gp.partials + (size_t)(d.mb + m) * N + n;
      float sum = 0.f;
      int sp = 0;
      for (; sp + 8 <= gp.splits; sp += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
          v[u] = __hip_atomic_load(src + (size_t)(sp + u) * sstride, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += v[u];
      }
      for (; sp < gp.splits; ++sp)
        sum += __hip_atomic_load(src + (size_t)sp * sstride, __ATOMIC_RELAXED,
                                 __HIP_MEMORY_SCOPE_AGENT);
      return sum;
    };
    if constexpr (FUSE) {
      // the tile holds tile_cols / 2 gate columns and as many up columns
      const int half_cols = d.tile_cols >> 1;
      const int items = d.mloc * half_cols;
      for (int idx = d.tid; idx < items; idx += d.nthreads) {
        const int m = idx / half_cols;
        const int n = d.tile * half_cols + (idx - m * half_cols);
        const uint16_t g = finish_output<DTYPE>(total(m, n), p.bias, n);
        const uint16_t u = finish_output<DTYPE>(total(m, half_n + n), p.bias, half_n + n);
        y[(size_t)(d.mb + m) * half_n + n] = act_mul<DTYPE>(g, u, p.gate_up_act - 1);
      }
    } else {
      // Up to four output elements per thread and pass, their loads all in flight: the partials
      // come from the memory side (they bypass the L2), so every pass of a thread costs a round
      // trip.  The sum of an element runs in split order whatever the grouping.
      const int items = d.mloc * d.tile_cols;
      const int nbase = d.tile * d.tile_cols;
      auto reduce = [&](auto iu_tag) {
        constexpr int IU = decltype(iu_tag)::value;
        constexpr int SU = IU == 1 ? 8 : 4;  // splits in flight per element
        for (int base = d.tid; base < items; base += IU * d.nthreads) {
          const float* src[IU];
          int row[IU], col[IU];
#pragma unroll
          for (int u = 0; u < IU; ++u) {
            const int idx = min(base + u * d.nthreads, items - 1);
            row[u] = idx / d.tile_cols;
            col[u] = nbase + (idx - row[u] * d.tile_cols);
            src[u] = gp.partials + (size_t)(d.mb + row[u]) * N + col[u];
          }
          float sum[IU] = {};
          int sp = 0;
          for (; sp + SU <= gp.splits; sp += SU) {
            float v[IU][SU];
#pragma unroll
            for (int s = 0; s < SU; ++s)
#pragma unroll
              for (int u = 0; u < IU; ++u)
                v[u][s] = __hip_atomic_load(src[u] + (size_t)(sp + s) * sstride, __ATOMIC_RELAXED,
                                            __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int s = 0; s < SU; ++s)
#pragma unroll
              for (int u = 0; u < IU; ++u) sum[u] += v[u][s];
          }
          for (; sp < gp.splits; ++sp) {
            float v[IU];
#pragma unroll
            for (int u = 0; u < IU; ++u)
              v[u] = __hip_atomic_load(src[u] + (size_t)sp * sstride, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
            for (int u = 0; u < IU; ++u) sum[u] += v[u];
          }
#pragma unroll
          for (int u = 0; u < IU; ++u)
            if (base + u * d.nthreads < items)
              y[(size_t)(d.mb + row[u]) * N + col[u]] = finish_output<DTYPE>(sum[u], p.bias, col[u]);
        }
      };
      if (items <= d.nthreads) reduce(std::integral_constant<int, 1>{});
      else if (items <= 2 * d.nthreads) reduce(std::integral_constant<int, 2>{});
      else reduce(std::integral_constant<int, 4>{});
    }
    if (d.tid == 0) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int DTYPE, int NT, int RMAX, bool FUSE = false, bool KQROWS = false>
__device__ __forceinline__ void gemv_finish(const GemvParams& gp, const Decomp& d, float (&out)[NT][RMAX], int col0,
                                            unsigned char* smem, PhaseStamps& ps) {
  gemv_finish_impl<DTYPE, NT, RMAX, FUSE, KQROWS>(gp, d, out, col0, smem, ps);
  ps.flush(gp, d);
}
template <int DTYPE, int NT, int RMAX, bool FUSE = false, bool KQROWS = false>
__device__ __forceinline__ void gemv_finish(const GemvParams& gp, const Decomp& d, float (&out)[NT][RMAX], int col0,
                                            unsigned char* smem) {
  PhaseStamps ps;
  gemv_finish_impl<DTYPE, NT, RMAX, FUSE, KQROWS>(gp, d, out, col0, smem, ps);
}

// ---------------------------------------------------------------------------------------
// GPTQ, contiguous groups.
// GSTEPS: MFMA steps (32 rows) per quantisation group inside a chunk: 1, 2 or 4.
// STATIC128: groupsize is exactly 128, so every chunk is one whole group.
// WORDS: adjacent packed words (columns) per lane: 4, 2 or 1, i.e. column tiles of 64, 32
// or 16 per wave.  Narrow tiles give enough workgroups to fill the chip without splitting
// K across workgroups, which removes the cross-workgroup reduction tail of small layers.
// FUSE (WORDS = 8): gated-MLP epilogue, W = [gate | up] along N.  The lane's eight words are
// four neighbouring gate columns and the four up columns N/2 further (two 128-bit loads per
// packed row); a wave covers 64 gate and 64 up columns, and the activation and the product
// happen in the lane that owns both sums.
// MOE: grouped launch, blockIdx.z is the expert; its rows (at most 16 per row block) and its
// tensors are found through gp.moe, workgroups of experts without rows leave at once.
template <int DTYPE, int RMAX, int GSTEPS, bool STATIC128, int WORDS, bool FUSE = false, bool MOE = false>
__global__ __launch_bounds__(512) void gemv_gptq_kernel(GemvParams gp) {
  static_assert(FUSE == (WORDS == 8), "eight words per lane = four gate + four up columns (fused only)");
  extern __shared__ __align__(16) unsigned char smem[];
  PhaseStamps ps;
  const int32_t* moe_rows = nullptr;
  if constexpr (MOE) {
    if (!moe_enter_decode(gp, moe_rows, FUSE)) return;
  }
  const Problem& p = gp.p;
  const Decomp d = make_decomp(gp, 16 * WORDS);
  const int N = p.N;
  // lane's first column (fused: its first gate column)
  const int nl = FUSE ? d.tile * (d.tile_cols >> 1) + d.wc * 64 + 4 * d.j
                      : d.tile * d.tile_cols + d.wc * 16 * WORDS + WORDS * d.j;
  const size_t up_cols = (size_t)(N >> 1);  // distance from a gate column to its up column
  const int nchunks = d.KW / kChunkRows;
  constexpr int GPC = kChunkSteps / GSTEPS;  // groups per chunk
  constexpr int PF = kPrefetch * 4 / WORDS;  // chunks in flight: same bytes for every WORDS

  SlabStager<true> slab;
  slab.issue(gp, d, moe_rows);

  // ---- issue the first PF chunks of weight loads.  Addresses are a wave-uniform 64-bit
  // base plus a per-lane 32-bit byte offset.
  const char* wbase = (const char*)(p.qweight + (size_t)(d.kw0 / 8) * N);
  const uint32_t w_lane = ((uint32_t)d.kq * (uint32_t)N + (uint32_t)nl) * 4u;
  const size_t step_bytes = (size_t)N * 16;  // four packed rows
  const uint32_t s_lane = (uint32_t)nl * 2u;
  const uint32_t z_lane = (uint32_t)(nl >> 3) * 4u;
  const int zshift = (nl & 7) * 4;
  struct Words { uint32_t v[WORDS]; };
  struct Scales { uint32_t v[(WORDS + 1) / 2]; };  // WORDS fp16 scales
  struct Zeros { uint32_t v[FUSE ? 2 : 1]; };      // packed zero points (fused: gate, up)
  Words wq[PF][kChunkSteps];
  Scales sc[PF][GPC];
  Zeros zw[PF][GPC];
  auto load_words = [&](const char* addr) {
    Words r;
    if constexpr (FUSE) {
      const uint4_t g = __builtin_nontemporal_load((const uint4_t*)addr);
      const uint4_t u = __builtin_nontemporal_load((const uint4_t*)(addr + up_cols * 4));
      r.v[0] = g.x; r.v[1] = g.y; r.v[2] = g.z; r.v[3] = g.w;
      r.v[4] = u.x; r.v[5] = u.y; r.v[6] = u.z; r.v[7] = u.w;
    } else if constexpr (WORDS == 4) {
      const uint4_t t = __builtin_nontemporal_load((const uint4_t*)addr);
      r.v[0] = t.x; r.v[1] = t.y; r.v[2] = t.z; r.v[3] = t.w;
    } else if constexpr (WORDS == 2) {
      const uint2_t t = __builtin_nontemporal_load((const uint2_t*)addr);
      r.v[0] = t.x; r.v[1] = t.y;
    } else {
      r.v[0] = __builtin_nontemporal_load((const uint32_t*)addr);
    }
    return r;
  };
  auto load_chunk = [&](int c, Words (&w)[kChunkSteps], Scales (&s)[GPC], Zeros (&z)[GPC]) {
#pragma unroll
    for (int st = 0; st < kChunkSteps; ++st)
      w[st] = load_words(wbase + (size_t)(c * kChunkSteps + st) * step_bytes + w_lane);
#pragma unroll
    for (int g = 0; g < GPC; ++g) {
      int gi = (d.kw0 + c * kChunkRows + g * GSTEPS * 32) / p.groupsize;
      gi = min(gi, p.num_groups - 1);
      const char* sp = (const char*)p.scales + (size_t)gi * N * 2 + s_lane;
      if constexpr (FUSE) {
        const uint2_t tg = *(const uint2_t*)sp;
        const uint2_t tu = *(const uint2_t*)(sp + up_cols * 2);
        s[g].v[0] = tg.x; s[g].v[1] = tg.y; s[g].v[2] = tu.x; s[g].v[3] = tu.y;
      } else if constexpr (WORDS == 4) {
        const uint2_t t = *(const uint2_t*)sp;
        s[g].v[0] = t.x; s[g].v[1] = t.y;
      } else if constexpr (WORDS == 2) {
        s[g].v[0] = *(const uint32_t*)sp;
      } else {
        s[g].v[0] = *(const uint16_t*)sp;
      }
      const char* zp = (const char*)p.qzeros + (size_t)gi * (N >> 3) * 4 + z_lane;
      z[g].v[0] = *(const uint32_t*)zp;
      if constexpr (FUSE) z[g].v[1] = *(const uint32_t*)(zp + (up_cols >> 3) * 4);
    }
  };
#pragma unroll
  for (int b = 0; b < PF; ++b)
    if (b < nchunks) load_chunk(b, wq[b], sc[b], zw[b]);
  ps.mark(6);

  slab.store(gp, d, smem);
  __syncthreads();
  ps.mark(1);

  const bool row_live = d.j < d.mloc;  // A-operand row of this lane
  // RMAX = 8: a second block of 16 activation rows takes the same unpacked weights
  constexpr bool ROWS32 = RMAX == 8;
  constexpr int R1 = RMAX < 4 ? RMAX : 4;  // live accumulator slots of the first block
  const bool row_live2 = ROWS32 && 16 + d.j < d.mloc;
  const unsigned char* a_base =
      smem + (size_t)d.j * gp.slab_stride + (size_t)(d.kwo + d.kq * 8) * 2;

  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  float4_t tot[WORDS], acc[WORDS];
  float4_t tot2[ROWS32 ? WORDS : 1], acc2[ROWS32 ? WORDS : 1];
#pragma unroll
  for (int t = 0; t < WORDS; ++t) tot[t] = acc[t] = zero4;
  if constexpr (ROWS32) {
#pragma unroll
    for (int t = 0; t < WORDS; ++t) tot2[t] = acc2[t] = zero4;
  }
  half2_t czlo[WORDS], czhi[WORDS];
  const SpliceConsts splice = splice_consts();

  auto process_chunk = [&](int c, const Words (&w)[kChunkSteps], const Scales (&s)[GPC],
                           const Zeros (&z)[GPC]) {
    const int kc = d.kw0 + c * kChunkRows;
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
        // (N/2 is a multiple of 8, so the up columns sit at the same nibbles of their word)
        const uint32_t z4 = gptq_zero_plus_one(z[gi].v[0]) >> zshift;
        uint32_t z4u = 0;
        if constexpr (FUSE) z4u = gptq_zero_plus_one(z[gi].v[1]) >> zshift;
#pragma unroll
        for (int t = 0; t < WORDS; ++t) {
          const uint32_t zz = FUSE && t >= 4 ? (z4u >> (4 * (t - 4))) & 0xFu : (z4 >> (4 * t)) & 0xFu;
          czlo[t] = as_half2(0xE400E400u | zz | (zz << 16));        // -(1024 + z)
          czhi[t] = as_half2(0xD400D400u | (zz << 4) | (zz << 20));  // -(64 + z)
        }
      }
      uint4_t a = {0u, 0u, 0u, 0u};
      if (row_live) a = *(const uint4_t*)(a_base + (size_t)(c * kChunkRows + st * 32) * 2);
      uint4_t a2 = {0u, 0u, 0u, 0u};
      if constexpr (ROWS32) {
        if (row_live2) a2 = *(const uint4_t*)(a_base + (size_t)16 * gp.slab_stride + (size_t)(c * kChunkRows + st * 32) * 2);
      }
#pragma unroll
      for (int t = 0; t < WORDS; ++t) {
        half2_t b[4];
        unpack_word_f16(w[st].v[t], czlo[t], czhi[t], splice, b);
        if (first && kStaticGroups) {
          acc[t] = mfma16<DTYPE>(a, b, zero4);
          if constexpr (ROWS32) acc2[t] = mfma16<DTYPE>(a2, b, zero4);
        } else {
          if (first && group_start) acc[t] = zero4;
          acc[t] = mfma16<DTYPE>(a, b, acc[t]);
          if constexpr (ROWS32) {
            if (first && group_start) acc2[t] = zero4;
            acc2[t] = mfma16<DTYPE>(a2, b, acc2[t]);
          }
        }
      }
      if (last && (kStaticGroups || group_end)) {
#pragma unroll
        for (int t = 0; t < WORDS; ++t) {
          const half2_t pr = as_half2(s[gi].v[t >> 1]);
          const float sf = (float)((t & 1) ? pr.y : pr.x);
#pragma unroll
          for (int r = 0; r < R1; ++r) tot[t][r] = fmaf(sf, acc[t][r], tot[t][r]);
          if constexpr (ROWS32) {
#pragma unroll
            for (int r = 0; r < 4; ++r) tot2[t][r] = fmaf(sf, acc2[t][r], tot2[t][r]);
          }
        }
      }
    }
  };

  // ring of PF chunk buffers: consume slot b, then refill it with chunk c + PF
  for (int c0 = 0; c0 < nchunks; c0 += PF) {
#pragma unroll
    for (int b = 0; b < PF; ++b) {
      const int c = c0 + b;
      if (c < nchunks) {
        process_chunk(c, wq[b], sc[b], zw[b]);
        if (c == 0) ps.mark_after(2, tot[0][0]);
        if (c + PF < nchunks) load_chunk(c + PF, wq[b], sc[b], zw[b]);
      }
    }
  }
  ps.mark_after(3, tot[0][0]);

  float out[WORDS][RMAX];
#pragma unroll
  for (int t = 0; t < WORDS; ++t)
#pragma unroll
    for (int r = 0; r < RMAX; ++r) {
      if constexpr (ROWS32) out[t][r] = r < 4 ? tot[t][r & 3] : tot2[t][r & 3];
      else out[t][r] = tot[t][r];
    }
  gemv_finish<DTYPE, WORDS, RMAX, FUSE>(gp, d, out, nl, smem, ps);
}

// ---------------------------------------------------------------------------------------
// GPTQ with g_idx (act-order), fp16.  LDS: [slab][g_idx slice as uint16][table G x tile_cols].
// Table entry (g, column) = fp16 scale | fp16 -(1024 + zero) << 16.
// XDIRECT: no activation slab.  A lane fetches the 16 bytes of its (row, K block) per 32-row step
// from global memory (the activations stay in L2) beside its weight words, so the LDS a
// workgroup needs does not grow with the rows: this kernel is bound by the per-weight work,
// not by memory, and what it wants is resident waves.
template <int DTYPE, int RMAX, bool MOE = false, bool XDIRECT = false>
__global__ __launch_bounds__(MOE ? 512 : 1024, 4) void gemv_gptq_act_kernel(GemvParams gp) {
  static_assert(!(MOE && XDIRECT), "grouped launches stage their (mapped) rows in LDS");
  extern __shared__ __align__(16) unsigned char smem[];
  const int32_t* moe_rows = nullptr;
  if constexpr (MOE) {
    if (!moe_enter_decode(gp, moe_rows)) return;
  }
  const Problem& p = gp.p;
  const Decomp d = make_decomp(gp, 64);
  const int N = p.N;
  const int nl = d.tile * d.tile_cols + d.wc * 64 + 4 * d.j;
  const int nsteps = d.KW / 32;
  constexpr int PF = 2;  // 32-row steps of weight loads in flight per wave

  const bool row_live = d.j < d.mloc;
  SlabStager<true> slab;
  if constexpr (!XDIRECT) slab.issue(gp, d, moe_rows);
  // XDIRECT: the lane's activations of a step, issued ahead of the weight words they meet
  // (memory returns in issue order: an L2 hit must not queue behind the weight stream)
  const uint16_t* x_lane = (const uint16_t*)p.x + (size_t)(d.mb + (row_live ? d.j : 0)) * p.K + d.kw0 + d.kq * 8;
  uint4_t aq[PF] = {};
  auto load_x = [&](int st) {
    uint4_t v = {0u, 0u, 0u, 0u};
    if (row_live) v = *(const uint4_t*)(x_lane + st * 32);
    return v;
  };

  const char* wbase = (const char*)(p.qweight + (size_t)(d.kw0 / 8) * N);
  const uint32_t w_lane = ((uint32_t)d.kq * (uint32_t)N + (uint32_t)nl) * 4u;
  const size_t step_bytes = (size_t)N * 16;
  uint4_t wq[PF];
  auto load_step = [&](int st) {
    return __builtin_nontemporal_load((const uint4_t*)(wbase + (size_t)st * step_bytes + w_lane));
  };
#pragma unroll
  for (int b = 0; b < PF; ++b)
    if (b < nsteps) {
      if constexpr (XDIRECT) aq[b] = load_x(b);
      wq[b] = load_step(b);
    }

  if constexpr (!XDIRECT) slab.store(gp, d, smem);

  // ---- g_idx slice of this workgroup, clamped to the table, as uint16; four entries per
  // thread and load, up to four loads in flight (a loop of dependent single loads costs one
  // memory round trip per iteration: 14 of them for a 7168-row range)
  uint16_t* gidx_s = (uint16_t*)(smem + gp.slab_bytes);
  constexpr int PU = 4;
  {
    const int32_t* gsrc = p.g_idx + d.kwg0;
    const int quads = d.KR >> 2;
    const int gmax = p.num_groups - 1;
    for (int i0 = d.tid; i0 < quads; i0 += PU * d.nthreads) {
      uint4_t v[PU];
#pragma unroll
      for (int u = 0; u < PU; ++u) {
        const int i = i0 + u * d.nthreads;
        if (i < quads) v[u] = *(const uint4_t*)(gsrc + 4 * i);
      }
#pragma unroll
      for (int u = 0; u < PU; ++u) {
        const int i = i0 + u * d.nthreads;
        if (i < quads) {
          const uint32_t g0 = (uint32_t)min(max((int)v[u].x, 0), gmax), g1 = (uint32_t)min(max((int)v[u].y, 0), gmax);
          const uint32_t g2 = (uint32_t)min(max((int)v[u].z, 0), gmax), g3 = (uint32_t)min(max((int)v[u].w, 0), gmax);
          *(uint2_t*)(gidx_s + 4 * i) = uint2_t{g0 | (g1 << 16), g2 | (g3 << 16)};
        }
      }
    }
  }
  // ---- scale / zero table of the workgroup's columns, all groups
  uint32_t* table = (uint32_t*)(smem + gp.slab_bytes + ((gp.kr_max * 2 + 15) & ~15));
  const int tc = d.tile_cols;
  uint32_t zref, zdiff;
  {
    const int nbase = d.tile * tc;
    const int words_per_row = tc >> 3;  // one qzeros word covers 8 columns
    const int items = p.num_groups * words_per_row;
    zref = gptq_zero_plus_one(p.qzeros[nbase >> 3]);
    zdiff = zref ^ ((zref & 0xFu) * 0x11111111u);
    for (int i0 = d.tid; i0 < items; i0 += PU * d.nthreads) {
      uint32_t zr[PU];
      uint4_t sr[PU];
#pragma unroll
      for (int u = 0; u < PU; ++u) {
        const int i = i0 + u * d.nthreads;
        if (i < items) {
          const int g = i / words_per_row;
          const int c8 = i - g * words_per_row;
          zr[u] = p.qzeros[(size_t)g * (N >> 3) + (nbase >> 3) + c8];
          sr[u] = *(const uint4_t*)(p.scales + (size_t)g * N + nbase + c8 * 8);
        }
      }
#pragma unroll
      for (int u = 0; u < PU; ++u) {
        const int i = i0 + u * d.nthreads;
        if (i < items) {
          const int g = i / words_per_row;
          const int c8 = i - g * words_per_row;
          const uint32_t z8 = gptq_zero_plus_one(zr[u]);
          zdiff |= z8 ^ zref;
          const uint32_t su[4] = {sr[u].x, sr[u].y, sr[u].z, sr[u].w};
          uint32_t e[8];
#pragma unroll
          for (int q = 0; q < 8; ++q) {
            const uint32_t s16 = (q & 1) ? (su[q >> 1] >> 16) : (su[q >> 1] & 0xFFFFu);
            const uint32_t z = (z8 >> (4 * q)) & 0xFu;
            e[q] = s16 | ((0xE400u | z) << 16);
          }
          uint4_t* dst = (uint4_t*)(table + (size_t)g * tc + c8 * 8);
          dst[0] = uint4_t{e[0], e[1], e[2], e[3]};
          dst[1] = uint4_t{e[4], e[5], e[6], e[7]};
        }
      }
    }
  }
  // One zero point for every group and column of the tile (symmetric quantization, the usual
  // companion of act-order): the zero pair of a weight pair is then a constant and its byte
  // permute drops out of the loop below (16 of ~137 vector instructions per 32-row step).
  const bool one_zero = __syncthreads_or((int)(zdiff != 0u)) == 0;
  const uint32_t c_const = 0xE400E400u | (zref & 0xFu) | ((zref & 0xFu) << 16);

  const unsigned char* a_base =
      smem + (size_t)d.j * gp.slab_stride + (size_t)(d.kwo + d.kq * 8) * 2;
  const uint16_t* g_base = gidx_s + d.kwo + d.kq * 8;
  const unsigned char* t_lane = (const unsigned char*)(table + d.wc * 64 + 4 * d.j);
  // a table row is 64 or 128 columns of 4 bytes: group -> byte offset is a shift (a 32-bit
  // integer multiply issues at a quarter of the rate)
  const int row_shift = __builtin_ctz((unsigned)tc) + 2;

  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  float4_t acc[4] = {zero4, zero4, zero4, zero4};
  const SpliceConsts splice = splice_consts();

  auto process_step = [&](int st, const uint4_t w, const uint4_t xa, auto one_zero_c) {
    constexpr bool ONE_ZERO = decltype(one_zero_c)::value;
    uint4_t a = {0u, 0u, 0u, 0u};
    if constexpr (XDIRECT) {
      // K order [0,4,1,5,2,6,3,7] of the splice
      a.x = __builtin_amdgcn_perm(xa.z, xa.x, 0x05040100u);
      a.y = __builtin_amdgcn_perm(xa.z, xa.x, 0x07060302u);
      a.z = __builtin_amdgcn_perm(xa.w, xa.y, 0x05040100u);
      a.w = __builtin_amdgcn_perm(xa.w, xa.y, 0x07060302u);
    } else {
      if (row_live) a = *(const uint4_t*)(a_base + (size_t)st * 64);
    }
    // groups of the 8 rows of this lane's K block, then their table rows (4 columns each)
    const uint4_t g8 = *(const uint4_t*)(g_base + st * 32);
    const uint32_t gw[4] = {g8.x, g8.y, g8.z, g8.w};
    uint32_t e[8][4];
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      const uint32_t g = (r & 1) ? (gw[r >> 1] >> 16) : (gw[r >> 1] & 0xFFFFu);
      const uint4_t row = *(const uint4_t*)(t_lane + (g << row_shift));
      e[r][0] = row.x; e[r][1] = row.y; e[r][2] = row.z; e[r][3] = row.w;
    }
    const uint32_t words[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      uint32_t b[4];
#pragma unroll
      for (int pr = 0; pr < 4; ++pr) {
        // rows pr and pr + 4 of the K block share one splice (nibbles 16 bits apart)
        // one byte permute each: the low halves (scales) and the high halves (-(1024 + z))
        const uint32_t ea = e[pr][t], eb = e[pr + 4][t];
        const uint32_t c2 = ONE_ZERO ? c_const : __builtin_amdgcn_perm(eb, ea, 0x07060302u);
        const uint32_t q2 = ((words[t] >> (4 * pr)) & splice.mask_lo) | splice.magic;
        const half2_t dq = as_half2(q2) + as_half2(c2);  // exact q - z
        if constexpr (DTYPE == Q4_DTYPE_F16) {
          const uint32_t s2 = __builtin_amdgcn_perm(eb, ea, 0x05040100u);
          b[pr] = as_u32(dq * as_half2(s2));  // one fp16 rounding, as the reference
        } else {
          // bf16: the exact fp32 products (mixed-precision multiplies that read the fp16 halves
          // where they lie: no scale pair needed), rounded once by the packed convert
          // (the compiler would emit two converts and a multiply per weight instead)
          const uint32_t dqu = as_u32(dq);
          float2_t f;
          asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[0,0,0] op_sel_hi:[1,1,0]" : "=v"(f.x) : "v"(dqu), "v"(ea));
          asm("v_fma_mix_f32 %0, %1, %2, 0 op_sel:[1,0,0] op_sel_hi:[1,1,0]" : "=v"(f.y) : "v"(dqu), "v"(eb));
          b[pr] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2_t));
        }
      }
      // b is in K order [0,4,1,5,2,6,3,7], the order of the staged activations
      const uint4_t bu = {b[0], b[1], b[2], b[3]};
      if constexpr (DTYPE == Q4_DTYPE_F16)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), __builtin_bit_cast(half8_t, bu), acc[t], 0, 0, 0);
      else
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, bu), acc[t], 0, 0, 0);
    }
  };

  auto walk = [&](auto one_zero_c) {
    for (int s0 = 0; s0 < nsteps; s0 += PF) {
#pragma unroll
      for (int b = 0; b < PF; ++b) {
        const int st = s0 + b;
        if (st < nsteps) {
          process_step(st, wq[b], aq[b], one_zero_c);
          if (st + PF < nsteps) {
            if constexpr (XDIRECT) aq[b] = load_x(st + PF);
            wq[b] = load_step(st + PF);
          }
        }
      }
    }
  };
  if (one_zero) walk(std::true_type{});
  else walk(std::false_type{});

  float out[4][RMAX];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < RMAX; ++r) out[t][r] = acc[t][r];
  gemv_finish<DTYPE, 4, RMAX>(gp, d, out, nl, smem);
}

// ---------------------------------------------------------------------------------------
// AWQ layout.  Wave tile: 256 columns (32 packed words) x 32 rows per step; lane (j, kq)
// loads words [8 rows of K block kq][2 adjacent words] and owns the 16 adjacent columns
// starting at 8 * (first word of the wave + 2 j).
template <int DTYPE, int RMAX, bool MOE = false>
__global__ __launch_bounds__(512) void gemv_awq_kernel(GemvParams gp) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int32_t* moe_rows = nullptr;
  if constexpr (MOE) {
    if (!moe_enter_decode(gp, moe_rows)) return;
  }
  const Problem& p = gp.p;
  const Decomp d = make_decomp(gp, 256);
  const int N = p.N;
  const int NC = N >> 3;                                             // packed words per row
  const int cw = (d.tile * d.tile_cols + d.wc * 256) / 8 + 2 * d.j;  // first of this lane's 2 words
  const int col0 = cw * 8;
  const int nsteps = d.KW / 32;
  constexpr int PF = 3;  // 32-row steps (8 x 64-bit loads each) in flight per wave

  SlabStager<false> slab;
  slab.issue(gp, d, moe_rows);

  const char* wbase = (const char*)(p.qweight + (size_t)d.kw0 * NC);
  const uint32_t w_lane = ((uint32_t)(d.kq * 8) * (uint32_t)NC + (uint32_t)cw) * 4u;
  const size_t row_bytes = (size_t)NC * 4;
  uint2_t wq[PF][8];
  auto load_step = [&](int st, uint2_t (&w)[8]) {
#pragma unroll
    for (int r = 0; r < 8; ++r)
      w[r] = __builtin_nontemporal_load(
          (const uint2_t*)(wbase + (size_t)(st * 32 + r) * row_bytes + w_lane));
  };
#pragma unroll
  for (int b = 0; b < PF; ++b)
    if (b < nsteps) load_step(b, wq[b]);

  slab.store(gp, d, smem);
  __syncthreads();

  const bool row_live = d.j < d.mloc;
  const unsigned char* a_base =
      smem + (size_t)d.j * gp.slab_stride + (size_t)(d.kwo + d.kq * 8) * 2;

  const float4_t zero4 = {0.f, 0.f, 0.f, 0.f};
  float4_t acc[16];
  float tot[16][RMAX];
#pragma unroll
  for (int t = 0; t < 16; ++t) {
    acc[t] = zero4;
#pragma unroll
    for (int r = 0; r < RMAX; ++r) tot[t][r] = 0.f;
  }
  half2_t cz[2][8];  // per word h and nibble position: -(1024 + z) (even) or -(64 + z) (odd)
  const SpliceConsts splice = splice_consts();
  const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};

  auto flush = [&](int g) {
    // scales of the lane's 16 columns: position pos of word h is column 8h + awq_order(pos)
    const uint4_t* sp = (const uint4_t*)(p.scales + (size_t)g * N + col0);
    const uint4_t s0 = sp[0], s1 = sp[1];
    const uint32_t su[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int pos = 0; pos < 8; ++pos) {
        const int col = 8 * h + (((pos & 3) << 1) | (pos >> 2));
        const half2_t pr = as_half2(su[col >> 1]);
        const float sf = (float)((col & 1) ? pr.y : pr.x);
#pragma unroll
        for (int r = 0; r < RMAX; ++r)
          tot[h * 8 + pos][r] = fmaf(sf, acc[h * 8 + pos][r], tot[h * 8 + pos][r]);
      }
  };

  auto process_step = [&](int st, const uint2_t (&w)[8]) {
    const int k = d.kw0 + st * 32;
    const int g = min(k / p.groupsize, p.num_groups - 1);
    const bool group_start = (st == 0) || (k % p.groupsize == 0);
    const bool group_end = (st == nsteps - 1) || ((k + 32) % p.groupsize == 0);
    if (group_start) {
      const uint2_t zw = *(const uint2_t*)(p.qzeros + (size_t)g * NC + cw);
      const uint32_t zz[2] = {zw.x, zw.y};
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int pos = 0; pos < 8; ++pos) {
          const uint32_t z = (zz[h] >> (4 * pos)) & 0xFu;  // AWQ zero points are used as stored
          cz[h][pos] = (pos & 1) ? as_half2(0xD400D400u | (z << 4) | (z << 20))
                                 : as_half2(0xE400E400u | z | (z << 16));
        }
#pragma unroll
      for (int t = 0; t < 16; ++t) acc[t] = zero4;
    }
    uint4_t a = {0u, 0u, 0u, 0u};
    if (row_live) a = *(const uint4_t*)(a_base + (size_t)st * 64);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      half2_t b[8][4];  // [nibble position][row pair]
#pragma unroll
      for (int rp = 0; rp < 4; ++rp) {
        const uint32_t w0 = h == 0 ? w[2 * rp].x : w[2 * rp].y;
        const uint32_t w1 = h == 0 ? w[2 * rp + 1].x : w[2 * rp + 1].y;
#pragma unroll
        for (int by = 0; by < 4; ++by) {
          // byte `by` of both rows side by side: low nibble = position 2*by, high = 2*by + 1
          const uint32_t sel = 0x0C000C00u | (uint32_t)by | ((uint32_t)(4 + by) << 16);
          const uint32_t t2 = __builtin_amdgcn_perm(w1, w0, sel);
          b[2 * by][rp] = as_half2((t2 & splice.mask_lo) | splice.magic) + cz[h][2 * by];
          b[2 * by + 1][rp] =
              as_half2((t2 & splice.mask_hi) | splice.magic) * sixteenth + cz[h][2 * by + 1];
        }
      }
#pragma unroll
      for (int pos = 0; pos < 8; ++pos) acc[h * 8 + pos] = mfma16<DTYPE>(a, b[pos], acc[h * 8 + pos]);
    }
    if (group_end) flush(g);
  };

  for (int s0 = 0; s0 < nsteps; s0 += PF) {
#pragma unroll
    for (int b = 0; b < PF; ++b) {
      const int st = s0 + b;
      if (st < nsteps) {
        process_step(st, wq[b]);
        if (st + PF < nsteps) load_step(st + PF, wq[b]);
      }
    }
  }

  // accumulator (h, pos) is column 8h + awq_order(pos) of the lane's 16
  float out[16][RMAX];
#pragma unroll
  for (int h = 0; h < 2; ++h)
#pragma unroll
    for (int pos = 0; pos < 8; ++pos)
#pragma unroll
      for (int r = 0; r < RMAX; ++r)
        out[8 * h + (((pos & 3) << 1) | (pos >> 2))][r] = tot[h * 8 + pos][r];
  gemv_finish<DTYPE, 16, RMAX>(gp, d, out, col0, smem);
}

}  // namespace q4
