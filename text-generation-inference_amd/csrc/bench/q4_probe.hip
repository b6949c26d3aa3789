// Measurement aid of the benchmark, built into its own library (libq4probe.so): kernels that
// only read.  They give the time a launch of the decode kernel's shape needs when it does
// nothing but pull its weight bytes out of HBM, which is the floor the decode kernels are
// compared with.  Not part of libq4linear.so or of its header; nothing in the product calls them.
//
//   q4_probe_read(buf, bytes, pattern, n_words, workgroups, threads, unroll, wcol, sink, stream)
//     pattern 0  linear: `workgroups` contiguous ranges, 1 KB per wave instruction
//     pattern 1  the decode kernels' pattern on a [bytes / (4 n_words), n_words] matrix of packed
//                words: a wave reads 4 rows x 256 B per instruction and walks down the rows;
//                a workgroup holds wcol column waves x (threads / 64 / wcol) K waves,
//                workgroups = n_words / (64 wcol) * K splits
//     pattern 2  an empty kernel of the same grid (launch cost alone)
//     unroll (1, 2, 4, 8): 16-byte loads a lane keeps in flight.  sink: 4 bytes of device memory,
//     never written in practice.  Shapes that do not divide are rejected (-1).
//   q4_probe_lds(lane_unit, iters, workgroups, sink, stream)
//     every wave of `workgroups` workgroups of 1024 threads issues `iters` rounds of eight 128-bit
//     LDS reads, lane l at the 16-byte unit lane_unit[l] (64 device ints, each 0..2887): timed with
//     different maps it shows which lanes the LDS serves in the same pass.  Synchronizes the
//     stream once to validate the map.
//   q4_probe_last_error()  message of the last refused call on this thread
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

namespace q4 {

typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

// One workgroup per contiguous range; every wave instruction reads 1 KB of consecutive bytes.
template <int U>
__global__ __launch_bounds__(1024) void probe_read_linear_kernel(const uint4_t* __restrict__ p, size_t vec_per_wg, uint32_t* sink) {
  const uint4_t* base = p + (size_t)blockIdx.x * vec_per_wg;
  uint4_t acc = {0u, 0u, 0u, 0u};
  const size_t nt = blockDim.x;
  for (size_t i = threadIdx.x; i < vec_per_wg; i += nt * U) {
    uint4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(base + i + (size_t)u * nt);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1u;  // keeps the loads alive
}

// The decode kernels' pattern on a [rows, n_words] matrix of packed words: a wave load covers
// four rows x 64 words (256 B per row); wave (tile, column wave, K slot) walks `steps` such loads
// down the rows.  grid = ntiles * splits, block = 64 * wcol * wk.
template <int U>
__global__ __launch_bounds__(1024) void probe_read_tile_kernel(const uint32_t* __restrict__ p, int n_words, int wcol, int wk,
                                                               int steps, int ntiles, uint32_t* sink) {
  const int w = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int wc = w % wcol, wave = w / wcol;
  const int tile = blockIdx.x % ntiles, split = blockIdx.x / ntiles;
  const int col = (tile * wcol + wc) * 64 + (lane & 15) * 4;
  const size_t row0 = ((size_t)split * wk + wave) * steps * 4 + (lane >> 4);
  const uint4_t* q = (const uint4_t*)(p + row0 * n_words + col);
  const size_t stride = (size_t)n_words;  // uint4 units between loads: 4 rows * n_words / 4
  uint4_t acc = {0u, 0u, 0u, 0u};
  for (int s = 0; s < steps; s += U) {
    uint4_t v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = __builtin_nontemporal_load(q + (size_t)(s + u) * stride);
#pragma unroll
    for (int u = 0; u < U; ++u) acc ^= v[u];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1u;
}

__global__ void probe_empty_kernel(uint32_t* sink) {
  if (sink == nullptr) sink[0] = 1u;
}

// 128-bit LDS reads with a caller-chosen lane -> 16-byte unit map: every wave of a 1024-thread
// workgroup issues `iters` rounds of eight ds_read_b128 (one wait per round), lane l at unit
// map[l] (+ 144 units per read of the round).  Timed, it tells which lane-to-address patterns
// the LDS serves at full rate, i.e. which lanes share a pass.
__global__ __launch_bounds__(1024) void probe_lds_read_kernel(const int* __restrict__ map, int iters, uint32_t* sink) {
  extern __shared__ __align__(16) unsigned char probe_smem[];
  for (int i = threadIdx.x; i < 16384; i += 1024) ((uint32_t*)probe_smem)[i] = (uint32_t)i;
  __syncthreads();
  const uint32_t addr = (uint32_t)map[threadIdx.x & 63] * 16u;
  uint4_t acc = {0u, 0u, 0u, 0u};
  for (int it = 0; it < iters; ++it) {
    uint4_t v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v[u]) : "v"(addr), "n"(u * 2304));
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u];
  }
  if ((acc.x ^ acc.y ^ acc.z ^ acc.w) == 0x12345678u) sink[0] = 1u;  // keeps the reads alive
}

}  // namespace q4

using namespace q4;

namespace {
constexpr int Q4_OK = 0, Q4_ERR_INVALID_ARGUMENT = -1, Q4_ERR_LAUNCH = -4;
thread_local char g_probe_error[256] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_probe_error, sizeof(g_probe_error), fmt, ap);
  va_end(ap);
}
}  // namespace

extern "C" const char* q4_probe_last_error(void) { return g_probe_error; }

extern "C" int q4_probe_read(const void* buf, size_t bytes, int pattern, int n_words, int workgroups, int threads, int unroll,
                             int wcol, void* sink, void* stream) {
  hipStream_t st = (hipStream_t)stream;
  if (sink == nullptr || workgroups <= 0 || threads <= 0 || threads > 1024 || threads % 64 != 0) {
    set_error("q4_probe_read: needs a sink, a positive grid and a block of whole waves (<= 1024 threads)");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (pattern == 2) {
    hipLaunchKernelGGL(probe_empty_kernel, dim3(workgroups), dim3(threads), 0, st, (uint32_t*)sink);
    return hipGetLastError() == hipSuccess ? Q4_OK : Q4_ERR_LAUNCH;
  }
  if (buf == nullptr || (unroll != 1 && unroll != 2 && unroll != 4 && unroll != 8)) {
    set_error("q4_probe_read: needs a buffer and an unroll of 1, 2, 4 or 8");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  if (pattern == 0) {
    // every workgroup reads the same whole number of (threads x unroll) vector rounds
    const size_t round = (size_t)threads * unroll;
    const size_t vec_per_wg = bytes / 16 / workgroups / round * round;
    if (vec_per_wg == 0) {
      set_error("q4_probe_read: %zu bytes are less than one round of %d workgroups", bytes, workgroups);
      return Q4_ERR_INVALID_ARGUMENT;
    }
    auto launch = [&](auto k) { hipLaunchKernelGGL(k, dim3(workgroups), dim3(threads), 0, st, (const uint4_t*)buf, vec_per_wg, (uint32_t*)sink); };
    if (unroll == 1) launch(probe_read_linear_kernel<1>);
    else if (unroll == 2) launch(probe_read_linear_kernel<2>);
    else if (unroll == 4) launch(probe_read_linear_kernel<4>);
    else launch(probe_read_linear_kernel<8>);
  } else if (pattern == 1) {
    if (wcol < 1 || (threads / 64) % wcol != 0 || n_words <= 0 || n_words % (64 * wcol) != 0 ||
        bytes % ((size_t)n_words * 16) != 0) {
      set_error("q4_probe_read: tile pattern needs n_words %% (64 wcol) == 0, whole K waves and a whole number of four-row steps");
      return Q4_ERR_INVALID_ARGUMENT;
    }
    const int wk = threads / 64 / wcol;
    const int ntiles = n_words / (64 * wcol);
    const size_t steps_total = bytes / ((size_t)n_words * 16);
    if (workgroups % ntiles != 0) {
      set_error("q4_probe_read: %d workgroups are not a multiple of the %d column tiles", workgroups, ntiles);
      return Q4_ERR_INVALID_ARGUMENT;
    }
    const size_t slots = (size_t)(workgroups / ntiles) * wk;
    if (steps_total % slots != 0 || (steps_total / slots) % unroll != 0) {
      set_error("q4_probe_read: %zu row steps do not divide over %zu wave slots x unroll %d", steps_total, slots, unroll);
      return Q4_ERR_INVALID_ARGUMENT;
    }
    const int steps = (int)(steps_total / slots);
    auto launch = [&](auto k) { hipLaunchKernelGGL(k, dim3(workgroups), dim3(threads), 0, st, (const uint32_t*)buf, n_words, wcol, wk, steps, ntiles, (uint32_t*)sink); };
    if (unroll == 1) launch(probe_read_tile_kernel<1>);
    else if (unroll == 2) launch(probe_read_tile_kernel<2>);
    else if (unroll == 4) launch(probe_read_tile_kernel<4>);
    else launch(probe_read_tile_kernel<8>);
  } else {
    set_error("q4_probe_read: unknown pattern %d", pattern);
    return Q4_ERR_INVALID_ARGUMENT;
  }
  return hipGetLastError() == hipSuccess ? Q4_OK : Q4_ERR_LAUNCH;
}

extern "C" int q4_probe_lds(const int32_t* lane_unit, int iters, int workgroups, void* sink, void* stream) {
  if (lane_unit == nullptr || sink == nullptr || iters <= 0 || workgroups <= 0) {
    set_error("q4_probe_lds: needs a 64-entry device map, a sink, positive iterations and workgroups");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  // the caller keeps every unit below (65536 - 7 * 2304) / 16 - 1 = 2887: checked on a host copy
  int32_t host_map[64];
  if (hipMemcpyAsync(host_map, lane_unit, sizeof(host_map), hipMemcpyDeviceToHost, (hipStream_t)stream) != hipSuccess ||
      hipStreamSynchronize((hipStream_t)stream) != hipSuccess) {
    set_error("q4_probe_lds: cannot read the lane map");
    return Q4_ERR_INVALID_ARGUMENT;
  }
  for (int l = 0; l < 64; ++l) {
    if (host_map[l] < 0 || host_map[l] > 2887) {
      set_error("q4_probe_lds: lane %d maps to unit %d, outside 0..2887", l, host_map[l]);
      return Q4_ERR_INVALID_ARGUMENT;
    }
  }
  hipLaunchKernelGGL(q4::probe_lds_read_kernel, dim3(workgroups), dim3(1024), 65536, (hipStream_t)stream, lane_unit, iters,
                     (uint32_t*)sink);
  return hipGetLastError() == hipSuccess ? Q4_OK : Q4_ERR_LAUNCH;
}
