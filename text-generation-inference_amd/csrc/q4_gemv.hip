// Decode path, host side: kernel choice, work decomposition and launch.  The kernels are in
// q4_gemv_kernels.cuh.
#include <cmath>
#include <cstring>
#include <initializer_list>

#include "q4_gemv_kernels.cuh"

#ifdef Q4_PHASE_STAMPS
// Measurement builds only: where the decode kernels of the following launches leave their clock
// readings ([workgroups][waves][8] 64-bit values; nullptr switches the stamps off).
static unsigned long long* g_phase_stamps = nullptr;
extern "C" void q4_phase_stamps_target(void* device_buffer) { g_phase_stamps = (unsigned long long*)device_buffer; }
// waves per launch the target buffer has room for (8 readings of 8 bytes each); a launch with more
// waves leaves no stamps
extern "C" int q4_phase_stamps_slots(void) { return Q4_PHASE_STAMP_SLOTS; }
#endif

namespace q4host {

using q4::GemvParams;
using q4::Problem;

// fused gated-MLP instantiations live in their own translation unit (q4_gemv_gate_up.hip)
void launch_gemv_gate_up(const GemvParams& gp, int dtype, int rmax, bool static128, dim3 grid, dim3 block,
                         size_t smem, hipStream_t stream, bool grouped);
// instruction-lean contiguous-group kernel (q4_gemv_lean.hip)
void launch_gemv_lean(const GemvParams& gp, int dtype, int mp, dim3 grid, dim3 block, size_t smem, hipStream_t stream);
void launch_gemv_awq_diag(const GemvParams& gp, int dtype, int row_groups, dim3 grid, dim3 block, size_t smem, hipStream_t stream);

// GPTQ layout, contiguous groups of whole 128-row chunks: what the lean kernel takes
bool gemv_lean_supported(const q4_weight* w, int dtype) {
  (void)dtype;
  return w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr && w->groupsize >= 128 && w->groupsize % 128 == 0 &&
         w->K % 128 == 0 && w->N % 64 == 0;
}

static bool groupsize_ok_contiguous(int gs) {
  return gs == 32 || gs == 64 || (gs >= 128 && gs % 128 == 0);
}

bool gemv_supported(const q4_weight* w, int M, int dtype) {
  if (M < 1) return false;
  if (w->K % 128 != 0) return false;
  const long chunks = (M + q4::kRowsPerBlock - 1) / q4::kRowsPerBlock;
  if (chunks > 65535) return false;
  if (w->layout == Q4_LAYOUT_AWQ) {
    if (w->N % 256 != 0 || w->groupsize % 32 != 0) return false;
    if ((long)w->num_groups * w->groupsize < w->K) return false;
    return chunks * (w->N / 256) <= Q4_WORKSPACE_TICKET_BYTES / 4;
  }
  if (w->N % 64 != 0) return false;
  // one ticket per (row chunk, column tile); the narrowest tile of each kernel decides
  const long tile = w->g_idx != nullptr ? 64 : 16;
  if (chunks * (w->N / tile) > Q4_WORKSPACE_TICKET_BYTES / 4 && M > 16) return false;
  if (w->g_idx != nullptr) {
    // act-order: the table of all groups for 64 columns must fit LDS next to the g_idx slice of
    // a workgroup's K range (at most 16 chunks of 128 rows once K is split as far as it goes)
    return w->num_groups <= 65535 && (long)w->num_groups * 64 * 4 + 16 * 256 + 32 <= 150000;
  }
  if (!groupsize_ok_contiguous(w->groupsize)) return false;
  return (long)w->num_groups * w->groupsize >= w->K;
}

bool gemv_gate_up_supported(const q4_weight* w, int M, int dtype) {
  // the contiguous-group GPTQ kernel with groups of whole chunks; both halves of W in whole
  // 64-column wave tiles.  Measured on the Llama-3-8B gate_up projection against the plain
  // kernel followed by the elementwise kernel: 16.1 / 18.2 us at M = 1, 17.2 / 18.4 us at
  // M = 2, 19.6 / 19.3 us at M = 4, 26.0 / 22.4 us at M = 8 (the fused workgroups are twice
  // as wide and stage twice the activation slab), so the fused kernel is offered for one and
  // two rows.
  return w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr && w->groupsize >= 128 && w->N % 128 == 0 &&
         M <= 2 && gemv_supported(w, M, dtype);
}

// 17..20 rows on the contiguous-group kernel: one workgroup takes all of them (two MFMA row
// blocks per unpacked word) with the configuration of 16 rows, when its slab still fits.
// Measured against the GEMM / two 16-row workgroups at M = 17: 14336 x 4096 18.0 against
// 22.8 us, 4096 x 28672 21.8 / 29.0, 8192 x 8192 18.2 / 20.9, 8192 x 28672 45.6 / 49.8.  The
// slab, its staging and the partial sums grow with every row: once the slab forces more K
// splits than 16 rows take (4096 x 28672 from 19 rows, 14336 x 4096 from 21) the kernel
// loses (M = 24: 33.5 against 29.6 us, 29.5 against 23.2 us).
bool gemv_rows32_kernel(const q4_weight* w, int M) {
  return w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr && M > 16 && M <= 32 && w->groupsize >= 32;
}

bool gemv_rows32_supported(const q4_weight* w, int M) {
  if (!gemv_rows32_kernel(w, M) || M > 20) return false;
  if (!gemv_supported(w, 16, Q4_DTYPE_F16)) return false;
  const GemvConfig c = gemv_pick_config(w, 16, false);
  const long chunks = w->K / 128;
  const long kr = (chunks + c.splits - 1) / c.splits * 128;
  const long slab = (long)M * (kr * 2 + 16);
  if (slab > 150000) return false;
  // a slab that leaves room for one workgroup per CU, and more workgroups than CUs: two rounds
  // (8192 x 7168: 19.4 us at M = 17, 27.9 us at M = 20 against 18.4 us for the prefill kernel)
  const long wgs = (long)(w->N / (16 * c.words * c.wcol)) * c.splits;
  return !(slab > 75 * 1024 && wgs > 256);
}

static GemvConfig pick_config(const q4_weight* w, int M, bool gate_up, bool allow_lean);

// the plain call of q4_linear: any kernel of the family
GemvConfig gemv_pick_config(const q4_weight* w, int M) {
  GemvConfig c = pick_config(w, M, false, true);
  // AWQ layout, plain call, up to 8 rows: the kernel that feeds the stored words to the matrix
  // core (its MFMA count grows with the rows).  Same decomposition, us on MI355X, new / old:
  // 4096 x 14336 12.0 / 13.3 at M = 1, 13.2 / 15.3 at M = 2, 15.0 / 18.4 at M = 4, 21.1 / 21.4 at
  // M = 8, 35.6 / 27.6 at M = 16; 14336 x 4096 11.8 / 13.0, 13.1 / 15.3, 17.1 / 20.2, 22.8 / 23.0,
  // 37.8 / 31.0; 4096 x 4096 8.5 / 9.0, 9.8 / 10.7, 11.6 / 13.5, 16.0 / 16.2, 21.3 / 27.3.
  if (w->layout == Q4_LAYOUT_AWQ && c.rows_per_block == 16 && M <= 8) c.lean = 1;
  return c;
}
// the kernels with the gated-MLP epilogue, two row blocks or an expert dimension (no lean variant)
GemvConfig gemv_pick_config(const q4_weight* w, int M, bool gate_up) { return pick_config(w, M, gate_up, false); }

static GemvConfig pick_config_search(const q4_weight* w, int M, bool gate_up, bool allow_lean);

// The choice depends on the weight's shape fields and M only, and the search behind it costs
// several microseconds on large layers - as much as a decode kernel runs: a small per-thread,
// direct-mapped memo keeps it out of the eager launch path.
static GemvConfig pick_config(const q4_weight* w, int M, bool gate_up, bool allow_lean) {
  struct Key {
    int32_t K, N, groupsize, num_groups, layout, act, M, flags;
  };
  struct Entry {
    Key key;
    GemvConfig cfg;
    bool valid;
  };
  static thread_local Entry memo[128];
  const Key key{w->K, w->N, w->groupsize, w->num_groups, w->layout, w->g_idx != nullptr ? 1 : 0, M,
                (gate_up ? 1 : 0) | (allow_lean ? 2 : 0)};
  uint32_t h = 2166136261u;
  for (const int32_t v : {key.K, key.N, key.groupsize, key.num_groups, key.layout, key.act, key.M, key.flags}) h = (h ^ (uint32_t)v) * 16777619u;
  Entry& e = memo[(h ^ (h >> 15)) & 127u];
  if (e.valid && memcmp(&e.key, &key, sizeof(Key)) == 0) return e.cfg;
  const GemvConfig cfg = pick_config_search(w, M, gate_up, allow_lean);
  e.key = key;
  e.cfg = cfg;
  e.valid = true;
  return cfg;
}

static GemvConfig pick_config_search(const q4_weight* w, int M, bool gate_up, bool allow_lean) {
  // Measured on MI355X (Llama-3-8B shapes, M=1): narrow column tiles with 4 waves along K
  // per workgroup and about two workgroups per CU (512 in flight) is the best point; wider
  // workgroups start too slowly and more splits lengthen the reduction tail.  The
  // activation slab (rows x K/splits) must fit its share of LDS.
  GemvConfig c;
  c.words = 4;
  if (!gate_up && gemv_rows32_supported(w, M)) {
    c = pick_config(w, 16, false, false);
    c.rows_per_block = 32;
    return c;
  }
  const int rows = M < c.rows_per_block ? M : c.rows_per_block;
  const int mchunks = (M + c.rows_per_block - 1) / c.rows_per_block;
  const int chunks = w->K / 128;
  // Large layers (from 32 M weights on), plain epilogue, up to 16 rows: the instruction-lean
  // kernel.  Measured against the kernel below on MI355X (us, same box): 4096 x 28672 14.5 / 15.6
  // at M = 1, 15.3 / 17.1 at M = 4, 18.2 / 20.1 at M = 16; 14336 x 4096 9.8 / 10.0, 12.9 / 13.5,
  // 14.8 / 15.9.  On small layers (4096 x 4096, 4096 x 6144), which are bound by launch, first
  // access and the split-K combine, it measured 0.5 us slower and is not taken.
  if (allow_lean && !gate_up && M <= 16 && gemv_lean_supported(w, Q4_DTYPE_F16) && (long)w->K * w->N >= (1L << 25) && chunks >= 8) {
    c.lean = 1;
    const int n64 = w->N / 64;
    if (n64 >= 384 && w->N % 128 == 0) {
      // the column tiles alone fill the chip: two per workgroup, K whole
      c.wcol = 2;
      c.wk = (M >= 4 && chunks % 8 == 0) ? 8 : 4;
      c.splits = 1;
      // many rows: one slab per workgroup must fit LDS.  When K has to be split for that, four
      // column tiles of four waves share each slab (8192 x 28672: 38.7 / 37.6 -> 30.2 / 31.3 us at
      // M = 12 / 16, 5120 x 27648 at M = 16: 29.9 -> 23.0 us against two tiles of eight waves).
      if ((long)rows * ((long)w->K * 2 + 16) > 150000 && w->N % 256 == 0 && chunks >= 8) {
        c.wcol = 4;
        c.wk = 4;
      }
      while ((long)rows * ((long)w->K / c.splits * 2 + 16) > 150000 && c.splits * c.wk * 2 <= chunks) c.splits *= 2;
      // From four rows on, a grid that spills into a second round it leaves mostly empty is handed
      // to the cost model below: 296 such workgroups of 3584 x 37888 hold a 115 KB slab each at
      // M = 16, one per CU (30.7 us; 25.9 us in 148 workgroups of four column tiles).  Elsewhere the
      // model's picks for these layers measured no better than the rule's (6144 x 24576 at M = 16:
      // 15 % slower).
      if (M < 4) return c;
      const long lds = (long)rows * ((long)((chunks + c.splits - 1) / c.splits) * 256 + 16) + 512;
      long res = (160 * 1024) / (lds + 1024);
      if (res > 16 / (c.wcol * c.wk)) res = 16 / (c.wcol * c.wk);
      if (res < 1) res = 1;
      const long wgs = (long)(n64 / c.wcol) * c.splits;
      const long rounds = ((wgs + 255) / 256 + res - 1) / res;
      if (rounds < 2 || wgs * 4 >= rounds * res * 256 * 3) return c;
    }
    const bool wide = n64 >= 384 && w->N % 128 == 0;
    int best = 1;
    double best_cost = -1.0;
    if (!wide) {
      c.wcol = 1;
      c.wk = 8;
    }
    // about one workgroup per CU; every wave keeps its own activations: rows x K / splits x 2 B in all
    bool full_round = false;
    for (int dv = 1; !wide && dv * c.wk <= chunks && (long)n64 * dv <= 256; ++dv)
      if ((long)n64 * dv >= 192 && (long)rows * c.wk * ((long)((chunks + dv * c.wk - 1) / (dv * c.wk)) * 256 + 16) <= 150000)
        full_round = true;
    if (n64 >= 128 && chunks >= 64 && M <= 3) full_round = true;
    for (int dv = 1; !wide && dv * c.wk <= chunks; ++dv) {
      const long lds = (long)rows * c.wk * ((long)((chunks + dv * c.wk - 1) / (dv * c.wk)) * 256 + 16);
      if (lds > 150000) continue;
      const double wgs = (double)n64 * dv;
      // Where some split count fills three quarters of the CUs or more in one round, going beyond
      // one workgroup per CU lets the CUs that take one more decide and is charged as whole rounds
      // (18944 x 3584 at M = 1: 11.6 us in 224 workgroups, 13.3 us in 280, 11.7 us in 504;
      // 6144 x 6144: 8.6 us in 192, 10.1 us in 288), and so it is over a long K whose tiles cover
      // half the CUs (8192 x 10240 at M = 1: 12.8 us in 160 workgroups, 14.7 us in 320, 16.5 us in
      // 480).  A short K with fewer tiles than that keeps its round and a third (4096 x 11008 at
      // M = 3: 12.9 us in 344 workgroups, 14.3 us in 172).
      double cost = wgs > 256.0 ? (full_round ? ceil(wgs / 256.0) : wgs / 256.0) : 256.0 / wgs;
      if (chunks % (dv * c.wk) != 0) cost *= 1.1;
      if (best_cost < 0.0 || cost < best_cost) {
        best_cost = cost;
        best = dv;
      }
    }
    // 160 column tiles or more over a short K (up to 4096 rows), four rows or more: every split
    // costs more in partial sums than the idle CUs do (4096 x 11008, 172 tiles: 10.2 / 10.7 / 11.9 us
    // unsplit at M = 4 / 8 / 16 against 13.5 / 14.2 / 16.4 us with two splits)
    if (!wide && M >= 4 && n64 >= 160 && chunks <= 32 && (long)rows * c.wk * ((long)((chunks + c.wk - 1) / c.wk) * 256 + 16) <= 150000)
      best = 1;
    if (!wide) c.splits = best;
    if (M >= 4) {
      // Four rows and more: the activation staging (per wave with one column wave, one slab per
      // workgroup with several) decides how many workgroups a CU holds, and the rule above knows
      // neither that nor rounds.  A small cost model fitted to sweeps on MI355X (us) searches every
      // (column waves, K waves, splits): a launch floor, the 128-row x 64-column chunk-tiles the
      // busiest CU walks (0.19 us each, up to 15 % more when fewer than 16 waves are resident
      // there), 2.5 us per further round when its workgroups do not fit together, the staged
      // activation bytes, the barrier of a shared slab, the slow start of 1024-thread workgroups
      // and the split-K combine.  Its pick replaces the rule's only where it predicts 12 % or
      // more: below that its error decides (measured on 11 layer shapes x M = 4..16: every pick
      // with a smaller predicted gain was 10-23 % slower than the rule's; the ones taken are
      // 8192 x 10240 17.5 / 18.7 / 24.5 -> 15.2 / 17.2 / 20.6 us at M = 4 / 8 / 16 and
      // 28672 x 8192 38.8 / 34.2 / 47.6 -> 27.3 / 28.6 / 34.1 us at M = 6 / 8 / 16).
      auto model_us = [&](int wcol, int wk, int dv) -> double {
        if (n64 % wcol != 0 || wcol * wk > 16 || dv * wk > chunks) return -1.0;
        const bool wave_slab = wcol == 1 || rows <= 2;
        const int per_wave = (chunks + dv * wk - 1) / (dv * wk);
        const int per_wg = (chunks + dv - 1) / dv;
        const long lds = (wave_slab ? (long)rows * wcol * wk * (per_wave * 256 + 16) : (long)rows * (per_wg * 256 + 16)) + 512;
        if (lds > 150000) return -1.0;
        long res = (160 * 1024) / (lds + 1024);
        if (res > 16 / (wcol * wk)) res = 16 / (wcol * wk);
        if (res < 1) res = 1;
        const long wgs = (long)(n64 / wcol) * dv;
        const long per_cu = (wgs + 255) / 256;
        const long waves = (per_cu < res ? per_cu : res) * wcol * wk;
        const double occ = 1.0 + 0.3 * (waves < 16 ? 16 - waves : 0) / 16.0;
        const long rounds = (per_cu + res - 1) / res;
        double t = 3.5 + 0.19 * (double)per_cu * per_wave * wk * wcol * occ + 2.5 * (rounds - 1);
        t += 0.015 * (double)per_cu * rows * per_wg * 256 / 1024.0;
        if (!wave_slab) t += 1.5;
        if (wcol * wk > 8) t += 1.2;
        if (dv > 1) t += 2.0 + 0.3 * dv * (M / 16.0);
        return t;
      };
      // Nine rows and more, and no single round of one-column-wave workgroups whose per-wave
      // activations fit LDS: one round of 1024-thread workgroups, two column tiles x eight K
      // waves (four x four next) around one shared slab.  Swept at M = 16 (us, this / the rule's
      // choice): 13824 x 5120 16.9 / 21.3, 5120 x 13824 16.5 / 22.1, 8192 x 10240 19.5 / 24.6.
      if (rows >= 9 && !wide) {
        bool one_round = false;
        for (int dv = 1; dv * 8 <= chunks && (long)n64 * dv <= 256; ++dv)
          if ((long)rows * 8 * (((chunks + dv * 8 - 1) / (dv * 8)) * 256 + 16) + 512 <= 150000) one_round = true;
        if (!one_round) {
          for (int wcol = 2; wcol <= 4; wcol *= 2) {
            const int wk = 16 / wcol;
            if (n64 % wcol != 0 || wk > chunks) continue;
            int pick_dv = 0;
            double pick_cost = -1.0;
            for (int dv = 1; dv * wk <= chunks && (long)(n64 / wcol) * dv <= 256; ++dv) {
              if ((long)rows * (((chunks + dv - 1) / dv) * 256 + 16) + 512 > 150000) continue;
              const int per_wave = (chunks + dv * wk - 1) / (dv * wk);
              const double cost = 256.0 / ((double)(n64 / wcol) * dv) * ((double)per_wave * dv * wk / chunks);
              if (pick_cost < 0.0 || cost < pick_cost) {
                pick_cost = cost;
                pick_dv = dv;
              }
            }
            if (pick_dv > 0) {
              c.wcol = wcol;
              c.wk = wk;
              c.splits = pick_dv;
              return c;
            }
          }
        }
      }
      const double t_rule = (wide || best_cost >= 0.0) ? model_us(c.wcol, c.wk, c.splits) : -1.0;
      double best_t = -1.0;
      GemvConfig pick = c;
      for (int wcol = 1; wcol <= 4; wcol *= 2)
        for (int wk = 2; wk <= 16; wk *= 2)
          for (int dv = 1; dv <= 32; ++dv) {
            const double t = model_us(wcol, wk, dv);
            if (t >= 0.0 && (best_t < 0.0 || t < best_t)) {
              best_t = t;
              pick.wcol = wcol;
              pick.wk = wk;
              pick.splits = dv;
            }
          }
      if (best_t >= 0.0 && (t_rule < 0.0 || best_t < 0.88 * t_rule)) return pick;
    }
    if (wide || best_cost >= 0.0) return c;
    c.lean = 0;  // no split fits LDS: the kernel below, with its workgroup slab
  }
  // Small layers, 4 to 16 rows, K a multiple of 1024 from 2048 on: 32-column wave tiles (two words per lane)
  // in eight-wave workgroups, about one workgroup per CU (two up to 8 rows); tiles that fill
  // the chip on their own are not split.  Swept on MI355X against the rule below (us, new /
  // old): 4096 x 4096 8.1 / 8.5 at M = 4, 8.3 / 9.2 at M = 8, 8.4 / 9.9 at M = 9, 8.9 / 9.5 at
  // M = 16; 4096 x 6144 9.8 / 10.7 at M = 9, 10.5 / 11.9 at M = 16; 8192 x 1024 7.5 / 9.1,
  // 7.8 / 10.1, 8.3 / 9.5 at M = 4, 8, 16; 2048 x 8192 6.4 / 8.2, 7.1 / 8.2, 7.9 / 9.7.
  if (allow_lean && !gate_up && w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr && w->groupsize >= 128 &&
      w->groupsize % 128 == 0 && M >= 4 && M <= 16 && chunks % 8 == 0 && chunks >= 8 && w->N % 64 == 0 &&
      // (4096 x 6144 up to 8 rows: no better than the rule below)
      (M >= 9 || w->N <= 4096 || w->N / 32 >= 256) &&
      // K = 1024: the eight-wave tiles only, up to two rounds of them (1024 x 8192 6.8 / 7.2 / 8.3 ->
      // 4.9 / 5.2 / 5.8 us at M = 4 / 8 / 16, 1024 x 2048 6.5 -> 4.7 us; 1024 x 28672, 896 tiles: 8.3 -> 10.6 us)
      (chunks >= 16 || ((w->N / 32 >= 256 || w->N <= 2048) && w->N / 32 <= 512))) {
    const bool narrow = w->N / 32 >= 256 || w->N <= 2048;  // one 32-column tile per workgroup, eight waves along K
    GemvConfig t = c;
    t.words = 2;
    t.wcol = narrow ? 1 : 2;
    t.wk = narrow ? 8 : 4;
    const long tiles = w->N / (32 * t.wcol);
    const int per = chunks / t.wk;
    const double target = (M <= 8 && !narrow) ? 512.0 : 256.0;
    int pick = -1;
    double pick_cost = -1.0;
    for (int dv = 1; dv <= per; ++dv) {
      if (per % dv != 0) continue;
      if ((long)rows * ((long)w->K / dv * 2 + 16) > 150000) continue;  // the workgroup's slab
      const double wgs = (double)tiles * dv;
      if (tiles >= 256 && dv > 1) break;
      const double cost = wgs >= target ? wgs / target : 1.5 * target / wgs;
      if (pick_cost < 0.0 || cost < pick_cost) {
        pick_cost = cost;
        pick = dv;
      }
    }
    if (pick > 0) {
      t.splits = pick;
      // A few workgroups more than CUs: the CUs that take two decide, and when the slab leaves
      // room for one per CU they form a second, nearly empty round (3072 x 9216, 288 workgroups:
      // 10.8 / 11.9 / 17.9 us at M = 4 / 8 / 16).  One round of the lean kernel's 64-column tiles,
      // eight waves over the whole K with their own activations, takes 9.0 / 9.6 / 10.7 us - where
      // those tiles are half the CUs or more (8192 x 1280 has 20: 14 us against 7.9 us).
      const long wgs = tiles * pick;
      const int per_wave = (chunks + 7) / 8;
      if (wgs > 256 && (wgs + 255) / 256 * 256 * 2 > wgs * 3 && w->N / 64 >= 128 && w->N / 64 <= 256 &&
          (long)rows * 8 * (per_wave * 256 + 16) + 512 <= 150000) {
        GemvConfig l = c;
        l.lean = 1;
        l.wcol = 1;
        l.wk = 8;
        l.splits = 1;
        return l;
      }
      return t;
    }
  }
  c.wcol = 1;
  c.wk = chunks >= 4 ? 4 : (chunks >= 2 ? 2 : 1);
  // wide layers with many rows: two column tiles per workgroup halve the slab staging
  // (and at any M once the tiles alone are well over the CU count: 4096 x 28672 at M = 1
  // measured 16.7 against 17.0-17.8 us)
  if (w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr && w->N % 128 == 0 &&
      ((M >= 8 && w->N / 64 >= 256) || (M >= 12 && w->N / 64 >= 128) || w->N / 64 >= 384 ||
       // long K: the slab staging of a workgroup is long, two tiles share it (28672 x 8192:
       // 23.3 against 25.2 us at M = 1, 28.6 against 36.3 us at M = 8)
       (w->K >= 16384 && w->N / 64 >= 128)))
    c.wcol = 2;
  const bool act = w->layout == Q4_LAYOUT_GPTQ && w->g_idx != nullptr;
  if (act) {
    // Act-order: the kernel is bound by its per-weight table lookups (VALU + LDS), not by
    // memory, and keeps no activation slab (its lanes fetch their activations themselves), so
    // its LDS use - the table of all groups for 64 columns and the g_idx slice - is the same
    // for every M.  Eight waves along K share the table; the split count aims at two workgroups
    // per CU (512; 256 when the table leaves room for one) and is charged the imbalance of
    // its K deal.  Against a sweep of 7 layer shapes x M = 1, 4, 16 x every (column waves,
    // K waves, splits) on MI355X this rule is 4 % above the best measured configuration on
    // average (worst: 8192 x 10240 and 4096 x 11008 at M = 1, 11-12 %, where four-wave
    // workgroups in more splits win).
    c.wcol = 1;
    c.wk = chunks >= 8 ? 8 : c.wk;
    const long table1 = (long)w->num_groups * 64 * 4;
    const int tiles = (w->N / 64) * mchunks;
    auto lds_bytes = [&](int dv) { return (long)((chunks + dv - 1) / dv) * 256 + table1 + 32; };
    // Workgroups beyond what the chip holds at once wait for a second round, which costs a
    // third of a full one even when nearly empty (18944 x 3584 at M = 1, 56 column tiles: 16.5 us
    // in 9 splits, 504 workgroups, against 21.7 us in 10).
    // (One or two rows over a small table - short workgroups, next to no partial sums - take the
    // extra round lightly: 4096 x 22016 at M = 1 21.1 us in two splits, 688 workgroups, against 22.9 us
    // unsplit; at M = 16 27.1 against 24.3 us.)
    const double late = (M <= 2 && table1 <= 16 * 1024) ? 0.1 : 0.35;
    auto grid_cost = [late](double wgs, double slots) {
      if (wgs <= slots) return slots / wgs;
      const double full = floor(wgs / slots), rem = wgs - full * slots;
      return full + (rem > 0.0 ? late + (1.0 - late) * rem / slots : 0.0);
    };
    int best_dv = chunks / c.wk;
    int best_wk = c.wk;
    double best = -1.0;
    // a short K that deals out evenly over four waves but not over eight is also tried with four
    // (3584 x 4608 at M = 1: 8.4 us as 4 x 7 against 10.2 us as 8 x 3, ragged)
    const bool try4 = c.wk == 8 && chunks % 8 != 0 && chunks % 4 == 0 && chunks <= 32 && mchunks == 1;
    for (int wk = c.wk; wk >= (try4 ? 4 : c.wk); wk -= 4) {
      for (int dv = 1; dv <= chunks / wk; ++dv) {
        if (lds_bytes(dv) > 150000) continue;
        const double slots = (lds_bytes(dv) > 80 * 1024 ? 256.0 : 512.0) * (wk == 4 ? 2.0 : 1.0);
        double cost = grid_cost((double)tiles * dv, slots);
        const int per_wave = (chunks + dv * wk - 1) / (dv * wk);  // chunks of the busiest wave
        cost *= (double)per_wave * dv * wk / chunks;
        if (lds_bytes(dv) > 80 * 1024) cost *= 1.5;  // one workgroup per CU: half the waves to hide the lookups
        if (wk == 4) cost *= 1.1;             // twice the table builds
        if (best < 0.0 || cost <= best) {
          best = cost;
          best_dv = dv;
          best_wk = wk;
        }
      }
    }
    c.wk = best_wk;
    c.splits = best_dv;
    // One 1024-thread workgroup per CU - two column tiles x eight K waves around one table of 128
    // columns - where 200 to 256 such workgroups make one round and their decomposition costs no more:
    // half the table builds and half the splits of two 512-thread workgroups per CU (us at M = 1 /
    // 16: 14336 x 4096 14.5 / 18.3 against 16.2 / 20.3, 8192 x 10240 18.0 / 21.4 against 19.6 / 24.2,
    // level on 28672 x 8192 and 4096 x 28672).
    if (w->N % 128 == 0 && chunks >= 8) {
      const int tiles2 = (w->N / 128) * mchunks;
      int pick = 0;
      double pick_cost = -1.0;
      for (int dv = 1; dv * 8 <= chunks; ++dv) {
        if ((long)((chunks + dv - 1) / dv) * 256 + 2 * table1 + 32 > 150000) continue;
        const double wgs = (double)tiles2 * dv;
        if (wgs < 200.0 || wgs > 256.0) continue;  // a single round (4096 x 11008 in 344: 17.9 against 15.0 us)
        const int per_wave = (chunks + dv * 8 - 1) / (dv * 8);
        const double cost = (wgs >= 256.0 ? wgs / 256.0 : 256.0 / wgs) * ((double)per_wave * dv * 8 / chunks);
        if (pick_cost < 0.0 || cost <= pick_cost) {
          pick_cost = cost;
          pick = dv;
        }
      }
      if (pick > 0 && best >= 0.0 && pick_cost <= 1.02 * best) {
        c.wcol = 2;
        c.wk = 8;
        c.splits = pick;
      }
    }
    return c;
  }
  // many rows, one column tile per workgroup: eight waves along K share one activation slab
  // (M = 16: 4096 x 6144 12.1 against 14.9 us, 14336 x 4096 18.8 against 22.4 us)
  const bool contiguous = w->layout == Q4_LAYOUT_GPTQ && w->g_idx == nullptr;
  if (contiguous && !gate_up && M >= 12 && c.wcol == 1 && (chunks % 8 == 0 || chunks >= 32)) c.wk = 8;
  // Several 16-row blocks whose tiles outnumber the CUs while the unsplit slab leaves room for one
  // workgroup per CU: two column tiles share each slab, one round instead of two (M = 64:
  // 3072 x 5120 20.2 -> 15.5 us, 3584 x 4608 29.8 -> 16.7 us; M = 48: 2560 x 6144 23.2 us before)
  if (contiguous && !gate_up && mchunks > 1 && c.wcol == 1 && w->N % 128 == 0 &&
      (long)rows * ((long)w->K * 2 + 16) > 75 * 1024 && (long)(w->N / 64) * mchunks > 256) {
    c.wcol = 2;
    c.wk = 4;
  }
  // 192..256 column tiles, 2..11 rows: one round of eight-wave workgroups over the whole K,
  // nothing to combine (4096 x 14336: 10.9 against 11.1 us at M = 2, 12.7 against 14.1 us at
  // M = 8; 5120 x 13824: 11.9 / 12.6 and 14.2 / 15.4 us; with 172 tiles it does not pay)
  if (contiguous && !gate_up && M >= 2 && M < 12 && c.wcol == 1 && w->N / 64 >= 192 && w->N / 64 <= 256 &&
      chunks >= 8 && (long)w->K * (rows * 2) <= 150000 - 16L * rows) {
    c.wk = 8;
    c.splits = 1;
    return c;
  }
  // AWQ: eight waves along K share one activation slab from 8 rows on, from 4 rows on large
  // layers and at any M once K is long (14336 x 4096 at M = 1: 13.2 against 17.5 us;
  // 4096 x 14336 at M = 8: 25.3 against 28.2 us; 4096 x 4096 up to 4 rows keeps four waves and
  // eight splits: 13.9 against 15.8 us).  A K that does not deal out evenly over eight waves
  // stays with four at small M (11008 x 4096 at M = 1: 14.9 against 17.1 us).
  const bool awq8 = w->layout == Q4_LAYOUT_AWQ && chunks >= 8 &&
                    (M >= 8 || (M >= 4 && (long)chunks * w->N >= 32L * 8192) || (chunks >= 64 && chunks % 8 == 0));
  if (awq8) c.wk = 8;
  if (gate_up) {
    // a wave owns 64 gate and 64 up columns (twice the bytes of a plain wave): eight waves
    // along K keep the wave count, and with it the bytes in flight, of the plain kernel
    c.wcol = 1;
    c.words = 8;
    if (chunks % 8 == 0 || chunks >= 32) c.wk = 8;
  }
  const int per_wg = chunks / c.wk;      // most splits: one chunk per wave
  const int wave_cols = w->layout == Q4_LAYOUT_AWQ ? 256 : (gate_up ? 128 : 64);
  const int ntiles = (w->N / (wave_cols * c.wcol)) * mchunks;
  int target_wgs = M <= 8 ? 512 : 384;  // partial-sum traffic grows with M
  // a single fp16 row combines its splits with one atomic per element: more, shorter
  // workgroups pay (4096 x 6144: 7.7 us with 8 splits against 8.4 us with 4)
  const bool cheap_combine = M == 1 && w->layout == Q4_LAYOUT_GPTQ && !gate_up;
  if (cheap_combine) target_wgs = 768;
  if (gate_up) target_wgs = 256;        // 512-thread workgroups: one per CU
  // the targets count four-wave workgroups: one with two column tiles (eight waves) counts twice
  // (4096 x 14336 at M = 16, two tiles per workgroup: 16.6 us with two splits, 18.9 us with four)
  const int tile_units = ntiles * (gate_up ? 1 : c.wcol) * (((contiguous && !gate_up) || awq8) && c.wk == 8 ? 2 : 1);
  int want = (target_wgs + tile_units / 2) / tile_units;
  // tiles that fill the chip on their own are not split (4096 x 28672: 18.5 us with two
  // splits against 16.7 us with one)
  if (want < 1 || ntiles * c.wcol >= 256) want = 1;
  // long K: no wave walks more than ~1024 rows when the tiles leave room for more workgroups
  // (28672 x 8192 at M = 8: 41.7 us with seven splits, 46.2 us with four)
  else if (contiguous && !gate_up && want < w->K / (c.wk * 1024)) want = w->K / (c.wk * 1024);
  // The slab of a workgroup is rows x K / splits activations and may take most of the LDS (one
  // workgroup per CU then): splitting K only to make the slab smaller costs more -- partial
  // sums of every row through memory -- than the lost co-residency.  4096 x 28672 at M = 16:
  // 19.7 us unsplit with a 128 KB slab against 30.8 us with four splits; 5120 x 13824 at M = 16:
  // 16 us with two splits (80 KB) against 26.8 us with five.
  long lds_budget = 150000 - 16L * rows;
  const long per_row = (long)rows * 2;  // bytes per K row in LDS
  int max_splits = per_wg;  // every wave gets at least one 128-row chunk
  // up to three rows combine through one atomic per element, for at most 14 splits: beyond, the
  // ticket scheme takes over and costs more than the extra workgroups bring (8192 x 1280 at
  // M = 1: 8.8 us in 16 splits against 6.2 us in 8)
  if (M <= 3 && !gate_up && max_splits > 14) max_splits = 14;
  int min_splits = lds_budget > 0 ? (int)(((long)w->K * per_row + lds_budget - 1) / lds_budget) : max_splits;
  if (min_splits < 1) min_splits = 1;
  if (min_splits > max_splits) min_splits = max_splits;
  if (awq8) {
    // 512-thread workgroups, one resident per CU for most slab sizes: the grid is held to one
    // round of 256 and aims at all of it for up to 8 rows, at three quarters beyond (the
    // partial sums grow with M).  Fitted on a sweep of 13 layer shapes x M = 1..16 on MI355X:
    // within 1.3 % of the best measured configuration on average (28672 x 8192 at M = 8: 42
    // against 62 us with ten ragged splits; 8192 x 10240 at M = 1: 18.6 against 24.7 us).
    const double target = M <= 8 ? 256.0 : 192.0;
    int best_dv = min_splits;
    double best = -1.0;
    for (int dv = min_splits; dv <= max_splits; ++dv) {
      const double wgs = (double)ntiles * dv;
      if (wgs > 256.0 && dv > min_splits) break;
      double cost = wgs > target ? wgs / target : target / wgs;
      if (chunks % (dv * c.wk) != 0) cost *= 1.2;
      if (best < 0.0 || cost < best) {
        best = cost;
        best_dv = dv;
      }
    }
    c.splits = best_dv;
    return c;
  }
  // four AWQ waves: at most 448 workgroups (13824 x 5120 at M = 1: 18.4 us with 14 splits
  // against 22.8 us with 27)
  const int max_wgs = w->layout == Q4_LAYOUT_AWQ ? 448 : 1 << 30;
  // K is dealt out in 128-row chunks over splits x wk wave slots.  A count that divides the
  // chunks evenly is preferred; when none is near the wanted one (K = 11008: 86 chunks) the
  // slots differ by one chunk and the cost carries the imbalance.
  int best = -1;
  double best_cost = -1.0;
  for (int dv = min_splits; dv <= max_splits; ++dv) {
    if ((long)ntiles * dv > max_wgs && dv > min_splits) break;
    const long slots = (long)dv * c.wk;
    const double balance = (double)((chunks + slots - 1) / slots) * slots / chunks;  // >= 1
    // too few workgroups cost more than too many (13824 x 5120 at M = 16 wants five splits:
    // nine take 19.4 us, three 24 us)
    double cost = dv > want ? (double)dv / want : 1.5 * want / dv;
    cost *= balance;
    if (chunks % slots != 0) cost *= 1.25;
    if (best_cost < 0.0 || cost < best_cost) {
      best_cost = cost;
      best = dv;
    }
  }
  c.splits = best > 0 ? best : max_splits;
  return c;
}

template <typename Kernel>
static void launch_kernel(Kernel k, const GemvParams& gp, dim3 grid, dim3 block, size_t smem,
                          hipStream_t stream) {
  if (smem > 64 * 1024)
    (void)hipFuncSetAttribute((const void*)k, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
  hipLaunchKernelGGL(k, grid, block, smem, stream, gp);
}

template <int DTYPE, int RMAX>
static void launch_rmax(const q4_weight* w, const GemvParams& gp, int words, dim3 grid, dim3 block,
                        size_t smem, hipStream_t stream) {
  using namespace q4;
  const int gs = w->groupsize;
  if (w->layout == Q4_LAYOUT_AWQ) {
    launch_kernel(gemv_awq_kernel<DTYPE, RMAX>, gp, grid, block, smem, stream);
  } else if (w->g_idx != nullptr) {
    launch_kernel(gemv_gptq_act_kernel<DTYPE, RMAX, false, true>, gp, grid, block, smem, stream);
  } else if (gs == 128) {
    if (words == 4) launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 4, true, 4>, gp, grid, block, smem, stream);
    else if (words == 2) launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 4, true, 2>, gp, grid, block, smem, stream);
    else launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 4, true, 1>, gp, grid, block, smem, stream);
  } else if (gs > 128) {
    if (words == 4) launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 4, false, 4>, gp, grid, block, smem, stream);
    else if (words == 2) launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 4, false, 2>, gp, grid, block, smem, stream);
    else launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 4, false, 1>, gp, grid, block, smem, stream);
  } else if (gs == 64) {
    launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 2, false, 4>, gp, grid, block, smem, stream);
  } else {
    launch_kernel(gemv_gptq_kernel<DTYPE, RMAX, 1, false, 4>, gp, grid, block, smem, stream);
  }
}

// 32 rows per workgroup: contiguous-group kernel, 64-column waves
template <int DTYPE>
static void launch_rows32(const q4_weight* w, const GemvParams& gp, dim3 grid, dim3 block, size_t smem,
                          hipStream_t stream) {
  using namespace q4;
  const int gs = w->groupsize;
  if (gs == 128) launch_kernel(gemv_gptq_kernel<DTYPE, 8, 4, true, 4>, gp, grid, block, smem, stream);
  else if (gs > 128) launch_kernel(gemv_gptq_kernel<DTYPE, 8, 4, false, 4>, gp, grid, block, smem, stream);
  else if (gs == 64) launch_kernel(gemv_gptq_kernel<DTYPE, 8, 2, false, 4>, gp, grid, block, smem, stream);
  else launch_kernel(gemv_gptq_kernel<DTYPE, 8, 1, false, 4>, gp, grid, block, smem, stream);
}

int launch_gemv(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype,
                void* workspace, size_t workspace_bytes, const GemvConfig* cfg_in,
                hipStream_t stream, int gate_up_act, const int32_t* x_perm) {
  using namespace q4;
  if (gate_up_act != 0 && !gemv_gate_up_supported(w, M, dtype)) {
    set_error("q4_linear_gate_up(gemv): no fused decode kernel for this weight (layout=%d g_idx=%p N=%d groupsize=%d)",
              w->layout, (const void*)w->g_idx, w->N, w->groupsize);
    return Q4_ERR_UNSUPPORTED;
  }
  if (!gemv_supported(w, M, dtype)) {
    set_error("q4_linear(gemv): unsupported problem (layout=%d g_idx=%p M=%d K=%d N=%d groupsize=%d dtype=%d)",
              w->layout, (const void*)w->g_idx, M, w->K, w->N, w->groupsize, dtype);
    return Q4_ERR_UNSUPPORTED;
  }
  // Up to sixteen fp16 rows on contiguous GPTQ groups, plain call: the short-launch kernel in
  // the decomposition of gemv_direct_default (which leaves the wide projections with more than
  // four rows to the kernels below).  Same-box A/B on MI355X against the kernels below, us at
  // M = 1 / 4 / 16: 4096 x 4096 5.33 / 7.90 / 8.81 -> 4.33 / 5.17 / 6.71, 4096 x 6144
  // 5.91 / 8.62 / 10.38 -> 5.00 / 5.93 / 8.29, 14336 x 4096 9.33 / 12.41 / 13.67 -> 8.12 / 9.50 /
  // 13.03, 4096 x 28672 13.55 / 16.71 -> 12.65 / 14.9 (16 rows: not taken).
  if (cfg_in == nullptr && gate_up_act == 0 && x_perm == nullptr && M <= 16 && dtype == Q4_DTYPE_F16) {
    int wk = 0, splits = 0;
    if (gemv_direct_default(w, M, dtype, &wk, &splits))
      return launch_gemv_direct(w, x, bias, y, M, dtype, workspace, workspace_bytes, wk, splits, stream);
  }
  const bool awq = w->layout == Q4_LAYOUT_AWQ;
  const bool act = !awq && w->g_idx != nullptr;
  GemvConfig cfg = cfg_in ? *cfg_in : (gate_up_act != 0 ? gemv_pick_config(w, M, true) : gemv_pick_config(w, M));
  const bool contiguous = !awq && !act;
  if (!contiguous || w->groupsize < 128) cfg.words = 4;  // only the contiguous-group kernel has narrow tiles
  if (gate_up_act != 0) cfg.words = 8;                    // four gate + four up words per lane
  if (cfg.words != 1 && cfg.words != 2 && cfg.words != 4 && !(cfg.words == 8 && gate_up_act != 0)) {
    set_error("q4_linear(gemv): words per lane must be 1, 2 or 4 (got %d)", cfg.words);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  const int wave_cols = awq ? 256 : 16 * cfg.words;
  const bool diag = awq && cfg.lean != 0 && gate_up_act == 0 && M <= 8;  // AWQ: words straight into the MFMA
  const bool lean = !awq && cfg.lean != 0;
  if (lean && !(gate_up_act == 0 && cfg.words == 4 && cfg.rows_per_block == 16 && gemv_lean_supported(w, dtype))) {
    set_error("q4_linear(gemv): the lean kernel takes GPTQ weights with contiguous groups of a multiple of 128 rows");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (cfg.wcol < 1 || cfg.wk < 1 || cfg.splits < 1 || cfg.wcol * cfg.wk > ((lean || act) ? 16 : 8) ||
      w->N % (wave_cols * cfg.wcol) != 0 || w->K % 128 != 0 || (long)cfg.splits * cfg.wk > w->K / 128) {
    set_error("q4_linear(gemv): bad config wcol=%d wk=%d splits=%d for K=%d N=%d", cfg.wcol, cfg.wk,
              cfg.splits, w->K, w->N);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (w->g_idx != nullptr && (cfg.wcol & (cfg.wcol - 1)) != 0) {
    set_error("q4_linear(gemv): the act-order kernel takes 1, 2 or 4 column waves (wcol=%d)", cfg.wcol);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (cfg.rows_per_block != 16 && !(cfg.rows_per_block == 32 && contiguous && gate_up_act == 0 && cfg.words == 4)) {
    set_error("q4_linear(gemv): %d rows per workgroup need the contiguous-group kernel with 64-column waves",
              cfg.rows_per_block);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  const int rpb = cfg.rows_per_block;
  const int rows = M < rpb ? M : rpb;
  const int mchunks = (M + rpb - 1) / rpb;
  // largest K range of a workgroup: K goes out in 128-row chunks over splits x wk wave slots
  GemvParams gp;
  const int KR = q4::set_k_deal(gp, w->K / 128, cfg.splits, cfg.wk);
  // the lean kernel gives every wave its own piece of LDS for the K range it walks
  const bool wave_slab = lean && (cfg.wcol == 1 || rows <= 2);
  const int slab_stride = (wave_slab ? q4::max_wave_rows(gp) : KR) * 2 + 16;
  // accumulator rows per lane: rows 4 kq .. 4 kq + 3 of an MFMA block (AWQ words-as-stored
  // kernel: rows kq, kq + 4, ..)
  const int rmax = diag ? (rows <= 4 ? 1 : 2) : (rpb == 32 ? 8 : (M <= 1 ? 1 : (M <= 2 ? 2 : 4)));
  const int nt = awq ? 16 : cfg.words;
  // act-order: no slab, the lanes fetch their activations themselves
  const bool x_direct = act;
  const size_t slab_bytes = x_direct ? 0 : ((size_t)rows * slab_stride * (wave_slab ? cfg.wcol * cfg.wk : 1) + 15) & ~(size_t)15;
  size_t smem = slab_bytes + (lean ? 512 : 0);  // lean: a block of zeros behind the slab
  if (act) smem += (((size_t)KR * 2 + 15) & ~(size_t)15) + (size_t)w->num_groups * 64 * cfg.wcol * 4;
  const size_t red = (size_t)(cfg.wk - 1) * cfg.wcol * nt * rmax * 64 * sizeof(float);
  if (red > smem) smem = red;
  const int ntiles = w->N / (wave_cols * cfg.wcol);
  if ((long)ntiles * mchunks > Q4_WORKSPACE_TICKET_BYTES / 4) {
    set_error("q4_linear(gemv): too many tiles (%d x %d)", ntiles, mchunks);
    return Q4_ERR_UNSUPPORTED;
  }
  float* partials = nullptr;
  uint32_t* tickets = nullptr;
  if (cfg.splits > 1) {
    const size_t need = Q4_WORKSPACE_COUNTER_BYTES + (size_t)cfg.splits * M * w->N * sizeof(float);
    if (workspace == nullptr || workspace_bytes < need) {
      set_error("q4_linear(gemv): workspace of %zu bytes needed, %zu given", need, workspace_bytes);
      return Q4_ERR_WORKSPACE;
    }
    tickets = (uint32_t*)workspace;
    partials = (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES);
  }
  gp.p = Problem{w->qweight, w->qzeros, (const half_t*)w->scales, w->g_idx, x, bias, y,
                 M,          w->K,      w->N,                     w->groupsize, w->num_groups};
  gp.p.gate_up_act = gate_up_act;
  gp.p.x_perm = x_perm;
  gp.partials = partials;
  gp.tickets = tickets;
  gp.wcol = cfg.wcol;
  gp.wk = cfg.wk;
  gp.splits = cfg.splits;
  // fp16, plain epilogue, at least four columns per lane: one atomic per element beats the
  // ticket.  The kernel first transposes a wave's sums through LDS (behind the K-wave partials)
  // so that an atomic instruction covers 64 consecutive cells of one row: issued straight from
  // the 16 lanes that hold a row, the four instructions of a GPTQ row cost 1 us more than the
  // one (4096 x 4096, M = 1: 7.05 against 5.97 us; tickets 7.8 us).  With several K waves the rows
  // are dealt to them (one round trip for all rows); a single K wave takes up to three rows in
  // turn, beyond that the tickets win.
  const int cell_rows_max = cfg.wk > 1 ? 16 : 3;
  gp.fixed_point_split = cfg.splits > 1 && cfg.splits <= 14 && dtype == Q4_DTYPE_F16 && gate_up_act == 0 &&
                         (nt >= 4 ? M <= cell_rows_max : M == 1) && (size_t)M * w->N * 8 <= Q4_WORKSPACE_CELL_BYTES;
  if (gp.fixed_point_split && nt >= 4) {
    const int tile_rows = diag ? (4 * rmax < kRowsPerBlock ? 4 * rmax : kRowsPerBlock) : (rmax < 4 ? rmax : kRowsPerBlock);
    const size_t tile = red + (size_t)cfg.wcol * tile_rows * 16 * nt * sizeof(float);
    if (tile > smem) smem = tile;
  }
  const size_t smem_limit = 160 * 1024 - 1024;  // gfx950: 160 KB of LDS per workgroup
  if (smem > smem_limit) {
    set_error("q4_linear(gemv): config needs %zu bytes of LDS (> %zu)", smem, smem_limit);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  gp.cells = cfg.splits > 1 ? (unsigned long long*)((char*)workspace + Q4_WORKSPACE_TICKET_BYTES) : nullptr;
  gp.slab_stride = slab_stride;
  gp.slab_bytes = (int)slab_bytes;
  gp.kr_max = KR;
  gp.partial_rows = M;
  gp.rows_per_block = rpb;
  gp.moe = q4::MoeView{};
  gp.ntiles = ntiles;
  gp.rows_per_block_alloc = rows;
  gp.wave_slab = wave_slab ? 1 : 0;
  dim3 grid((unsigned)(ntiles * cfg.splits), (unsigned)mchunks);
  dim3 block((unsigned)(64 * cfg.wcol * cfg.wk));
#ifdef Q4_PHASE_STAMPS
  gp.stamps = (long)grid.x * grid.y * (block.x >> 6) <= Q4_PHASE_STAMP_SLOTS ? g_phase_stamps : nullptr;
#endif
  if (diag) {
    launch_gemv_awq_diag(gp, dtype, rmax, grid, block, smem, stream);
  } else if (lean) {
    launch_gemv_lean(gp, dtype, rows <= 1 ? 1 : (rows <= 2 ? 2 : (rows <= 4 ? 4 : (rows <= 8 ? 8 : 16))), grid, block, smem,
                     stream);
  } else if (gate_up_act != 0) {
    launch_gemv_gate_up(gp, dtype, rmax, w->groupsize == 128, grid, block, smem, stream, false);
  } else if (rmax == 8) {
    if (dtype == Q4_DTYPE_F16) launch_rows32<Q4_DTYPE_F16>(w, gp, grid, block, smem, stream);
    else launch_rows32<Q4_DTYPE_BF16>(w, gp, grid, block, smem, stream);
  } else if (dtype == Q4_DTYPE_F16) {
    if (rmax == 1) launch_rmax<Q4_DTYPE_F16, 1>(w, gp, cfg.words, grid, block, smem, stream);
    else if (rmax == 2) launch_rmax<Q4_DTYPE_F16, 2>(w, gp, cfg.words, grid, block, smem, stream);
    else launch_rmax<Q4_DTYPE_F16, 4>(w, gp, cfg.words, grid, block, smem, stream);
  } else {
    if (rmax == 1) launch_rmax<Q4_DTYPE_BF16, 1>(w, gp, cfg.words, grid, block, smem, stream);
    else if (rmax == 2) launch_rmax<Q4_DTYPE_BF16, 2>(w, gp, cfg.words, grid, block, smem, stream);
    else launch_rmax<Q4_DTYPE_BF16, 4>(w, gp, cfg.words, grid, block, smem, stream);
  }
  hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemv): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
