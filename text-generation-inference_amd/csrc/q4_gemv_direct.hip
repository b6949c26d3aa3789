// Host side of the short-launch decode kernel (q4_gemv_direct.cuh): what it takes, and its launch.
#include "q4_gemv_direct.cuh"

#ifdef Q4_PHASE_STAMPS
static unsigned long long* g_direct_stamps = nullptr;
extern "C" void q4_phase_stamps_target_direct(void* device_buffer) { g_direct_stamps = (unsigned long long*)device_buffer; }
#endif

namespace q4host {

using q4::DirectParams;

// GPTQ layout, contiguous groups of 128 << s rows (or one group), K in whole chunks, N in whole
// 64-column tiles, tensors below 4 GB (32-bit buffer offsets); up to 16 rows; every (split, wave)
// slot walks at least one chunk.
bool gemv_direct_supported(const q4_weight* w, int M, int dtype, int wk, int splits) {
  (void)dtype;
  if (w->layout != Q4_LAYOUT_GPTQ || w->g_idx != nullptr || M < 1 || M > 16) return false;
  if (w->K % 128 != 0 || w->N % 64 != 0) return false;
  if (w->num_groups > 1) {
    const int per = w->groupsize / 128;
    if (w->groupsize % 128 != 0 || per < 1 || (per & (per - 1)) != 0) return false;
  }
  if ((long)w->num_groups * w->groupsize < w->K) return false;
  // 32-bit byte offsets; the lane offset of an activation row past M must not wrap either
  if ((long)(w->K / 8) * w->N * 4 >= (1L << 32) || (long)w->num_groups * w->N * 2 >= (1L << 32) || (long)16 * w->K * 2 >= (1L << 32))
    return false;
  if (wk < 1 || wk > 8 || splits < 1 || splits > 65535 || (long)wk * splits > w->K / 128) return false;
  // four chunks or more per wave: the loop variant marks refills past a wave's range with bit 31 of
  // the lane offset, so every tensor must end below 2 GB
  if ((w->K / 128 + wk * splits - 1) / (wk * splits) > 3 &&
      ((long)(w->K / 8) * w->N * 4 >= (1L << 31) || (long)w->num_groups * w->N * 2 >= (1L << 31) || (long)16 * w->K * 2 >= (1L << 31)))
    return false;
  if (splits > 1 && w->N / 64 > Q4_WORKSPACE_TICKET_BYTES / 4) return false;
  return true;
}

// K splits meet in the fixed-point cells (one atomic per output element) for fp16 rows and up to
// 14 splits while the rows' cells fit their part of the workspace; otherwise through fp32 partial
// sums and a ticket per column tile.
static bool direct_uses_cells(const q4_weight* w, int M, int dtype, int splits) {
  return splits > 1 && splits <= 14 && dtype == Q4_DTYPE_F16 && M <= 16 && (size_t)M * w->N * 8 <= Q4_WORKSPACE_CELL_BYTES;
}

size_t gemv_direct_workspace_bytes(const q4_weight* w, int M, int dtype, int splits) {
  if (splits <= 1) return 0;
  if (direct_uses_cells(w, M, dtype, splits)) return Q4_WORKSPACE_COUNTER_BYTES;
  return (size_t)Q4_WORKSPACE_COUNTER_BYTES + (size_t)splits * M * w->N * sizeof(float);
}

// The decomposition the plain call takes when it runs this kernel; false when the kernel does
// not take the problem, the splits would not meet in the cells, or the slab kernels are the
// better choice.
//   Up to two rows, and three or four rows on fewer than 256 column tiles: four K waves per
// workgroup (fewer on a K shorter than four chunks) and the fewest K splits, up to the 14 the
// cells count, that leave every wave the fewest chunks.
//   Three and four rows on 256 column tiles or more: four K waves, K whole (no atomics).
// Five to sixteen rows: eight K waves and the fewest splits that deal K evenly, leave a wave at
// most two chunks and make 192 workgroups or more (else the four-row rule).  With 256 column
// tiles or more (no split) and more than four rows every wave would re-read its share of the
// activations from L2 next to a long weight stream; the kernels that stage the activations once
// per workgroup are faster there (4096 x 28672, 16 rows: 19.8 against 17.5 us), so those shapes
// are not taken.
bool gemv_direct_default(const q4_weight* w, int M, int dtype, int* wk_out, int* splits_out) {
  const int chunks = w->K / 128;
  const int tiles = w->N / 64;
  // (sweep of the four Llama-3-8B projections at three and four rows, us, this rule against the
  // one-workgroup-per-CU rule it replaces there: 4096 x 6144 M = 4 5.92 / 7.05, 4096 x 4096 5.13 /
  // 5.52, 14336 x 4096 9.75 / 10.00; 4096 x 28672 M = 3 with K whole 14.35 against 16.19 in 8 splits)
  if (M <= 2 || (M <= 4 && tiles < 256)) {
    const int wk = chunks >= 4 ? 4 : (chunks >= 2 ? 2 : 1);
    if (!gemv_direct_supported(w, M, dtype, wk, 1)) return false;
    int best_s = 1, best = (chunks + wk - 1) / wk;
    for (int s = 2; s <= 14 && wk * s <= chunks; ++s) {
      const int per = (chunks + wk * s - 1) / (wk * s);
      if (per < best) {
        best = per;
        best_s = s;
      }
    }
    if (best_s > 1 && !direct_uses_cells(w, M, dtype, best_s)) return false;
    *wk_out = wk;
    *splits_out = best_s;
    return true;
  }
  if (tiles < 1 || (tiles >= 256 && M > 4)) return false;
  int s = tiles >= 256 ? 1 : (256 + tiles / 2) / tiles;
  s = s < 1 ? 1 : (s > 14 ? 14 : s);
  int wk = M > 4 ? 8 : 4;
  if (M > 4) {
    // the fewest splits that deal K evenly, leave a wave at most two chunks and make 192
    // workgroups or more (4096 x 6144: 8 x 2, 4096 x 4096: 8 x 4, 14336 x 4096: 8 x 7)
    for (int t = 1; t <= 14; ++t) {
      if (chunks % (8 * t) == 0 && chunks / (8 * t) <= 2 && (long)tiles * t >= 192) {
        s = t;
        break;
      }
    }
  }
  while (wk > 1 && wk * s > chunks) wk >>= 1;
  while (s > 1 && wk * s > chunks) --s;
  if (!gemv_direct_supported(w, M, dtype, wk, s)) return false;
  if (s > 1 && !direct_uses_cells(w, M, dtype, s)) return false;
  *wk_out = wk;
  *splits_out = s;
  return true;
}

template <int DTYPE, int MR>
static void launch_one(const DirectParams& dp, dim3 grid, dim3 block, size_t smem, hipStream_t stream) {
  // the straight-line variant when no wave walks more than three chunks
  if (dp.cpw + (dp.rem > 0 ? 1 : 0) <= 3) hipLaunchKernelGGL((q4::gemv_gptq_direct_kernel<DTYPE, MR, false>), grid, block, smem, stream, dp);
  else hipLaunchKernelGGL((q4::gemv_gptq_direct_kernel<DTYPE, MR, true>), grid, block, smem, stream, dp);
}

template <int DTYPE>
static void launch_dtype(const DirectParams& dp, int mr, dim3 grid, dim3 block, size_t smem, hipStream_t stream) {
  if (mr == 1) launch_one<DTYPE, 1>(dp, grid, block, smem, stream);
  else if (mr == 2) launch_one<DTYPE, 2>(dp, grid, block, smem, stream);
  else if (mr == 4) launch_one<DTYPE, 4>(dp, grid, block, smem, stream);
  else launch_one<DTYPE, 16>(dp, grid, block, smem, stream);
}

int launch_gemv_direct(const q4_weight* w, const void* x, const void* bias, void* y, int M, int dtype, void* workspace,
                       size_t workspace_bytes, int wk, int splits, hipStream_t stream) {
  if (!gemv_direct_supported(w, M, dtype, wk, splits)) {
    set_error("q4_linear(gemv, short-launch kernel): unsupported problem or decomposition (M=%d K=%d N=%d groupsize=%d wk=%d splits=%d dtype=%d)",
              M, w->K, w->N, w->groupsize, wk, splits, dtype);
    return Q4_ERR_UNSUPPORTED;
  }
  DirectParams dp;
  dp.qweight = w->qweight;
  dp.qzeros = w->qzeros;
  dp.scales = (const q4::half_t*)w->scales;
  dp.x = x;
  dp.bias = bias;
  dp.y = y;
  dp.cells = nullptr;
  dp.partials = nullptr;
  dp.tickets = nullptr;
  const size_t need = gemv_direct_workspace_bytes(w, M, dtype, splits);
  if (need > 0) {
    if (workspace == nullptr || workspace_bytes < need) {
      set_error("q4_linear(gemv): workspace of %zu bytes needed, %zu given", need, workspace_bytes);
      return Q4_ERR_WORKSPACE;
    }
    if (direct_uses_cells(w, M, dtype, splits)) {
      dp.cells = (unsigned long long*)((char*)workspace + Q4_WORKSPACE_TICKET_BYTES);
    } else {
      dp.tickets = (uint32_t*)workspace;
      dp.partials = (float*)((char*)workspace + Q4_WORKSPACE_COUNTER_BYTES);
    }
  }
  const int chunks = w->K / 128, slots = wk * splits;
  dp.N = w->N;
  dp.K = w->K;
  dp.M = M;
  dp.cpw = chunks / slots;
  dp.rem = chunks % slots;
  dp.gshift = 31;
  if (w->num_groups > 1) {
    dp.gshift = 0;
    while ((128 << dp.gshift) < w->groupsize) ++dp.gshift;
  }
  dp.num_groups = w->num_groups;
  dp.splits = splits;
  const int mr = M <= 1 ? 1 : (M <= 2 ? 2 : (M <= 4 ? 4 : 16));
  const dim3 grid((unsigned)(w->N / 64), (unsigned)splits);
  const dim3 block((unsigned)(64 * wk));
#ifdef Q4_PHASE_STAMPS
  dp.stamps = (long)grid.x * grid.y * wk <= Q4_PHASE_STAMP_SLOTS ? g_direct_stamps : nullptr;
#endif
  // every wave's activation chunk (up to four rows), the K waves' sums, then the ticket drawn
  const size_t smem = (mr <= 4 ? (size_t)wk * 1024 : 0) + (size_t)wk * mr * 64 * sizeof(float) + 16;
  if (dtype == Q4_DTYPE_F16) launch_dtype<Q4_DTYPE_F16>(dp, mr, grid, block, smem, stream);
  else launch_dtype<Q4_DTYPE_BF16>(dp, mr, grid, block, smem, stream);
  const hipError_t err = hipGetLastError();
  if (err != hipSuccess) {
    set_error("q4_linear(gemv, short-launch kernel): launch failed: %s", hipGetErrorString(err));
    return Q4_ERR_LAUNCH;
  }
  return Q4_OK;
}

}  // namespace q4host
