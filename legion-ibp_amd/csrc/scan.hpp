// Device-wide exclusive scan in three phases over fixed 2048-item tiles:
//   1. the producer kernel writes cnt[i] and one sum per tile (tile_reduce_store),
//   2. scan_tiles_kernel (one block) turns tile sums into tile offsets and
//      publishes the total,
//   3. scan_apply_kernel writes the exclusive prefix of every item.
// Item counts are read from device memory so no phase needs a host round-trip.
#pragma once

#include "device.hpp"

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
