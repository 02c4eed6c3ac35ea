// Device-wide exclusive scans, two kinds.
//
// On the per-batch path: a single-pass scan with decoupled look-back (ScanChain,
// scan_tile_prefix, further down) that lives inside the producing kernel, so a hop needs
// no scan launches of its own.
//
// At cache-build time, where launch count does not matter: a three-phase scan over fixed
// 2048-item tiles --
//   1. the producer kernel writes cnt[i] and one sum per tile (tile_reduce_store),
//   2. scan_tiles_kernel (one block) turns tile sums into tile offsets and
//      publishes the total,
//   3. scan_apply_kernel writes the exclusive prefix of every item.
// Item counts are read from device memory so no phase needs a host round-trip.
#pragma once

#include "device.hpp"
#include "lookback.hpp"

namespace lmi {

constexpr int kScanBlock = 256;
constexpr int kScanItems = 8;
constexpr int kScanTile = kScanBlock * kScanItems;  // 2048

// Block-wide sum of `v`; thread 0 stores it to tile_sums[tile].
__device__ __forceinline__ void tile_reduce_store(int v, int32_t *tile_sums, int tile, int *lds) {
#pragma unroll
  for (int d = kWave / 2; d > 0; d >>= 1) v += __shfl_down(v, d, kWave);
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  if (lane == 0) lds[wid] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    int t = 0;
#pragma unroll
    for (int w = 0; w < kScanBlock / kWave; ++w) t += lds[w];
    tile_sums[tile] = t;
  }
  __syncthreads();
}

// Header updates that ride on the scan total (thread 0 of the single block).
// Reference semantics: counter_update, engine/operator_impl.cu:58-91.
__device__ __forceinline__ void scan_epilogue(int epilogue, DevState *st, int hop, int total) {
  if (epilogue == SCAN_EPI_HOP_EDGES) {
    const int eoff = (hop == 0) ? 0 : st->edge_counter[12 + hop] + st->edge_counter[9 + hop];
    st->edge_counter[9 + hop + 1] = total;
    st->edge_counter[12 + hop + 1] = eoff;
    st->edge_counter[0] = eoff;
    st->edge_counter[1] = total;
  } else if (epilogue == SCAN_EPI_HOP_NODES) {
    const int n_prev = st->node_counter[9 + hop];
    st->node_counter[9 + hop + 1] = n_prev + total;
    st->node_counter[0] = st->node_counter[2] = st->node_counter[4] = n_prev;
    st->node_counter[1] = st->node_counter[3] = st->node_counter[5] = total;
    st->node_counter[7] = n_prev + total;
  }
}

static __global__ __launch_bounds__(1024) void scan_tiles_kernel(int32_t *tile_sums,
                                                                 const int32_t *n_ptr, int epilogue,
                                                                 DevState *st, int hop,
                                                                 int32_t *total_out) {
  __shared__ int lds[1024 / kWave + 1];
  const int n = *n_ptr;
  const int n_tiles = (n + kScanTile - 1) / kScanTile;
  int carry = 0;
  for (int base = 0; base < n_tiles; base += 1024) {
    const int t = base + threadIdx.x;
    const int v = (t < n_tiles) ? tile_sums[t] : 0;
    int total;
    const int ex = block_exclusive_scan<1024>(v, lds, total);
    if (t < n_tiles) tile_sums[t] = carry + ex;
    carry += total;
  }
  if (threadIdx.x == 0) {
    *total_out = carry;
    scan_epilogue(epilogue, st, hop, carry);
  }
}

static __global__ __launch_bounds__(kScanBlock) void scan_apply_kernel(const int32_t *cnt,
                                                                       const int32_t *tile_sums,
                                                                       const int32_t *n_ptr,
                                                                       const int32_t *total_ptr,
                                                                       int32_t *out) {
  __shared__ int lds[kScanBlock / kWave + 1];
  const int n = *n_ptr;
  const int n_tiles = (n + kScanTile - 1) / kScanTile;
  if (blockIdx.x == 0 && threadIdx.x == 0) out[n] = *total_ptr;
  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int base = tile * kScanTile + threadIdx.x * kScanItems;
    int v[kScanItems], sum = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
      v[j] = (base + j < n) ? cnt[base + j] : 0;
      sum += v[j];
    }
    int total;
    int run = block_exclusive_scan<kScanBlock>(sum, lds, total) + tile_sums[tile];
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
      if (base + j < n) out[base + j] = run;
      run += v[j];
    }
  }
}

// ---------------------------------------------------------------------------
// Single-pass scan (decoupled look-back, Merrill & Garland 2016) for the kernels on
// the per-batch path: the producer kernel itself turns its per-item counts into
// exclusive prefixes, so a hop needs one launch where the three-phase scan needs
// three.  One tile per block, tile = blockIdx.x: a tile only ever waits for
// lower-numbered blocks, which the dispatcher started earlier, and every block
// publishes its own sum before it looks back, so the wait always ends.  (An
// atomic ticket would drop the reliance on dispatch order, but 500 same-address
// atomics cost more than the whole scan.)  The wait is bounded all the same.
//
// status[t] = (flag << 32) | value in one 64-bit word, written and read with
// relaxed device-scope atomics (flag and value travel together, nothing else is
// exchanged): flag 0 = not ready, 1 = value is the tile's own sum, 2 = value is
// the inclusive prefix up to and including the tile.  The status words must be
// zeroed by an earlier kernel of the same stream before each use.
struct ScanChain {
  unsigned long long *status;  // [max_tiles]
};

constexpr unsigned long long kScanAggregate = 1ull << 32, kScanInclusive = 2ull << 32;
// A tile that waits longer than this for an earlier tile gives up, raises DevState::scan_fault
// (and the server's sticky fault word) and writes nothing.  Wall-clock ticks, not re-reads: a
// legitimate wait is microseconds, whatever else shares the device (wall_clock64 counts at a
// constant 100 MHz: a quarter of a second).  The clock is read once per 1024 re-reads.
constexpr long long kScanWaitTicks = 25000000;
constexpr int kScanFaultPrefix = -1;  // what scan_tile_prefix returns to a tile that gave up

// Zeroes a chain for a later kernel; call from any grid with a flat thread index.
__device__ __forceinline__ void scan_chain_reset(ScanChain c, int max_tiles, int64_t tid, int64_t n_threads) {
  for (int64_t i = tid; i < max_tiles; i += n_threads) c.status[i] = 0ull;
}

__device__ __forceinline__ void scan_publish(ScanChain c, int tile, unsigned long long word) {
  __hip_atomic_store(&c.status[tile], word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Publishes this tile's aggregate and returns the exclusive prefix of the tile
// (sum of all earlier tiles) to every thread of the block, or kScanFaultPrefix to every
// thread when the wait ran out: the tile then has no valid offset and must write nothing.
// Wavefront 0 looks back 64 tiles per step (lookback_window).  lds_prefix is one shared int.
// Contains __syncthreads.
__device__ __forceinline__ int scan_tile_prefix(ScanChain c, int tile, int aggregate, int *lds_prefix,
                                                DevState *st) {
  if (threadIdx.x < kWave) {
    const int lane = threadIdx.x;
    int prefix = 0;
    if (tile == 0) {
      if (lane == 0) scan_publish(c, 0, kScanInclusive | (unsigned int)aggregate);
    } else {
      if (lane == 0) scan_publish(c, tile, kScanAggregate | (unsigned int)aggregate);
      int base = tile - 1;
      int spins = 0;
      // after a first fault every later tile gives up almost at once, so a broken chain drains
      // in milliseconds
      const bool broken = st->scan_fault != 0;
      const long long t0 = wall_clock64();
      while (true) {
        const int j = base - lane;
        unsigned long long w = kScanInclusive;  // before tile 0: an inclusive prefix of 0
        if (j >= 0) w = __hip_atomic_load(&c.status[j], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        const unsigned flag = (unsigned)(w >> 32);
        const LookbackWindow win = lookback_window(__ballot(flag == 2u), __ballot(flag == 0u));
        if (win.wait) {  // a tile we need has not published yet: read again
          ++spins;
          const bool out_of_time = broken ? spins >= 64 : ((spins & 1023) == 0 && wall_clock64() - t0 > kScanWaitTicks);
          if (!out_of_time) continue;
          if (lane == 0) raise_fault(st, kFaultScan);  // never expected; bounded so that the grid always drains
          prefix = kScanFaultPrefix;
          break;
        }
        int contrib = ((win.take >> lane) & 1ull) ? (int)(unsigned)w : 0;
#pragma unroll
        for (int d = kWave / 2; d > 0; d >>= 1) contrib += __shfl_xor(contrib, d, kWave);
        prefix += contrib;
        if (win.done) break;
        base -= kWave;
      }
      if (lane == 0 && prefix != kScanFaultPrefix) scan_publish(c, tile, kScanInclusive | (unsigned int)(prefix + aggregate));
    }
    if (lane == 0) *lds_prefix = prefix;
  }
  __syncthreads();
  return *lds_prefix;
}

// Phases 2 and 3.  n_max bounds *n_ptr and sizes the apply grid.
static inline int launch_scan_phases(hipStream_t st, const int32_t *cnt, int32_t *out,
                                     int32_t *tile_sums, const int32_t *n_ptr, int64_t n_max,
                                     int epilogue, DevState *state, int hop, int32_t *total_out) {
  hipLaunchKernelGGL(scan_tiles_kernel, dim3(1), dim3(1024), 0, st, tile_sums, n_ptr, epilogue, state,
                     hop, total_out);
  int64_t tiles = ceil_div(n_max > 0 ? n_max : 1, kScanTile);
  int grid = (int)(tiles < 2048 ? tiles : 2048);
  hipLaunchKernelGGL(scan_apply_kernel, dim3(grid), dim3(kScanBlock), 0, st, cnt, tile_sums, n_ptr,
                     total_out, out);
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

static inline int scan_grid(int64_t n_max) {
  int64_t tiles = ceil_div(n_max > 0 ? n_max : 1, kScanTile);
  return (int)(tiles < 2048 ? tiles : 2048);
}

}  // namespace lmi
