// Seed staging and the per-hop sampling / dedup / relabel kernels.
//
// Reference semantics (Legion-IBP, sampling_server/src/engine/operator_impl.cu):
//   batch_generate :28-56    seeds become local ids 0..n-1 in batch order
//   random_sample  :178-302  hop k samples from ALL nodes known so far; a row with
//                            deg <= fanout is taken whole in CSR order; edges run
//                            neighbour -> node
//   construct_graph:304-317  edges relabelled to local ids
//   counter_update :58-91    16-int headers
// What differs on purpose: Philox4x32-10 keyed by (seed, hop, node, slot) with
// Floyd's without-replacement rule instead of a per-node default-seeded
// minstd_rand; an open-addressing hash table in HBM instead of an N-bit bitmap
// plus an N-entry position map; scans instead of atomics for placement, so the
// edge order is (node, slot) and local ids follow first occurrence in that order.
#include "scan.hpp"

namespace lmi {

// ------------------------------------------------------------ batch start
// Clears the dedup table (key = -1, value = INT_MAX), resets the pipe state and
// stores the per-batch parameters where the later kernels read them.
static __global__ __launch_bounds__(256) void batch_begin_kernel(HashSlot *slots, int64_t n_slots,
                                                                 DevState *st, int hops, BatchParams bp) {
  const int64_t tid = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // two slots (16 bytes) per store
  const int4 fill = make_int4(kEmptyKey, kIntMax, kEmptyKey, kIntMax);
  int4 *p = reinterpret_cast<int4 *>(slots);
  for (int64_t i = tid; i < n_slots / 2; i += stride) p[i] = fill;
  if (tid == 0) {
    int32_t *w = reinterpret_cast<int32_t *>(st);
    for (int i = 0; i < (int)(sizeof(DevState) / 4); ++i) w[i] = 0;
    st->node_counter[8] = hops;
    st->node_counter[9] = bp.n_seeds;
    st->node_counter[1] = st->node_counter[3] = st->node_counter[5] = bp.n_seeds;
    st->node_counter[7] = bp.n_seeds;
    st->rng_lo = (uint32_t)bp.rng_seed;
    st->rng_hi = (uint32_t)(bp.rng_seed >> 32);
    st->lru_tick = bp.lru_tick;
    st->n_seeds = bp.n_seeds;
    st->seeds = bp.seeds;
    st->labels_in = bp.labels;
  }
}

// Stage the seeds: ids[i] = seed, labels, and table[seed] = min(i) so that a
// repeated seed resolves to its first row.
static __global__ __launch_bounds__(256) void batch_generate_kernel(int64_t n_nodes, int32_t *ids, int32_t *labels,
                                                                    HashSlot *slots, int log2cap, DevState *st) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= st->n_seeds) return;
  const int32_t id = st->seeds[i];
  ids[i] = id;
  labels[i] = st->labels_in ? st->labels_in[i] : -1;
  if (id < 0 || id >= n_nodes) {
    st->bad_id = 1;
    return;
  }
  table_insert_min(slots, log2cap, id, i);
}

// ------------------------------------------------------------- hop, phase 1
// cnt[i] = min(deg(ids[i]), fanout) for every node known so far, plus tile sums.
static __global__ __launch_bounds__(kScanBlock) void hop_count_kernel(
    const int32_t *ids, const int64_t *indptr, int64_t n_nodes, int fanout, int hop, const DevState *st,
    int32_t *cnt, int32_t *tile_sums) {
  __shared__ int lds[kScanBlock / kWave];
  const int n = st->node_counter[9 + hop];
  const int n_tiles = (n + kScanTile - 1) / kScanTile;
  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int base = tile * kScanTile + threadIdx.x * kScanItems;
    int sum = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
      const int i = base + j;
      if (i < n) {
        const int32_t v = ids[i];
        int c = 0;
        if (v >= 0 && v < n_nodes) {
          const int64_t deg = indptr[v + 1] - indptr[v];
          c = (int)(deg < (int64_t)fanout ? deg : (int64_t)fanout);
        }
        cnt[i] = c;
        sum += c;
      }
    }
    tile_reduce_store(sum, tile_sums, tile, lds);
  }
}

// ------------------------------------------------------------- hop, phase 2
// One group of G lanes per node, one lane per output slot.  Rows no longer than
// the fanout are copied whole; longer rows draw `fanout` distinct positions with
// Floyd's rule, the group resolving collisions slot by slot through shuffles.
// Every sampled edge is inserted into the dedup table with candidate value
// n_prev + e (e = edge index inside the hop); atomicMin keeps the first edge.
template <int G>
static __global__ __launch_bounds__(256) void hop_sample_kernel(
    const int32_t *ids, const int64_t *indptr, const int32_t *indices, int64_t n_nodes, int fanout,
    int hop, const DevState *st, const int32_t *row_ptr, int32_t *agg_src_ids, int32_t *agg_dst_off,
    HashSlot *slots, int log2cap, int32_t *eslot) {
  const uint64_t seed = (uint64_t)st->rng_lo | ((uint64_t)st->rng_hi << 32);
  const int n_prev = st->node_counter[9 + hop];
  const int eoff = st->edge_counter[12 + hop + 1];
  const int lane = threadIdx.x & (G - 1);
  const int group = (blockIdx.x * blockDim.x + threadIdx.x) / G;
  const int n_groups = gridDim.x * blockDim.x / G;
  for (int i = group; i < n_prev; i += n_groups) {
    const int32_t v = ids[i];
    if (v < 0 || v >= n_nodes) continue;
    const int64_t beg = indptr[v];
    const int64_t deg = indptr[v + 1] - beg;
    const int base = row_ptr[i];
    int64_t pick = lane;
    int count;
    if (deg <= (int64_t)fanout) {
      count = (int)deg;
    } else {
      count = fanout;
      const uint32_t j = (uint32_t)(deg - fanout) + (uint32_t)lane;
      uint32_t t = 0xFFFFFFFFu;
      if (lane < fanout) t = __umulhi(sample_draw(seed, (uint32_t)hop, (uint32_t)v, (uint32_t)lane), j + 1u);
      bool dup = false;
      for (int q = 0; q + 1 < fanout; ++q) {
        const uint32_t mine = dup ? j : t;
        const uint32_t p = __shfl(mine, q, G);
        if (lane > q && t == p) dup = true;
      }
      pick = dup ? j : t;
    }
    if (lane < count) {
      const int32_t nbr = indices[beg + pick];
      const int e = base + lane;
      agg_src_ids[eoff + e] = nbr;
      agg_dst_off[eoff + e] = i;
      eslot[e] = (int)table_insert_min(slots, log2cap, nbr, n_prev + e);
    }
  }
}

// ------------------------------------------------------------- hop, phase 3
// firstv[e] = table value of the edge's source; an edge is the first occurrence
// of a new node iff that value names the edge itself.  cnt[e] = flag, tile sums.
static __global__ __launch_bounds__(kScanBlock) void hop_flag_kernel(
    const HashSlot *slots, const int32_t *eslot, int hop, const DevState *st, int32_t *firstv,
    int32_t *cnt, int32_t *tile_sums) {
  __shared__ int lds[kScanBlock / kWave];
  const int n_prev = st->node_counter[9 + hop];
  const int n = st->edge_counter[9 + hop + 1];
  const int n_tiles = (n + kScanTile - 1) / kScanTile;
  for (int tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int base = tile * kScanTile + threadIdx.x * kScanItems;
    int sum = 0;
#pragma unroll
    for (int j = 0; j < kScanItems; ++j) {
      const int e = base + j;
      if (e < n) {
        const int32_t val = slots[eslot[e]].val;
        firstv[e] = val;
        const int flag = (val == n_prev + e) ? 1 : 0;
        cnt[e] = flag;
        sum += flag;
      }
    }
    tile_reduce_store(sum, tile_sums, tile, lds);
  }
}

// ------------------------------------------------------------- hop, phase 4
// local id of an edge source: an old node keeps its id; a new node gets
// n_prev + (rank of its first edge among first edges).  First edges also
// append the node to ids[] and publish the final id in the table.
static __global__ __launch_bounds__(256) void hop_relabel_kernel(
    const int32_t *firstv, const int32_t *rank, const int32_t *eslot, int hop, const DevState *st,
    const int32_t *agg_src_ids, int32_t *agg_src_off, int32_t *ids, HashSlot *slots) {
  const int n_prev = st->node_counter[9 + hop];
  const int n = st->edge_counter[9 + hop + 1];
  const int eoff = st->edge_counter[12 + hop + 1];
  for (int e = blockIdx.x * blockDim.x + threadIdx.x; e < n; e += gridDim.x * blockDim.x) {
    const int32_t val = firstv[e];
    int32_t local = val;
    if (val >= n_prev) {
      local = n_prev + rank[val - n_prev];
      if (val == n_prev + e) {
        ids[local] = agg_src_ids[eoff + e];
        slots[eslot[e]].val = local;
      }
    }
    agg_src_off[eoff + e] = local;
  }
}

// ---------------------------------------------------------------- launchers
static void begin_args(Server *s, Pipe &p, const BatchParams &bp, void **args, HashSlot **slots, int64_t *n_slots,
                       DevState **st, int *hops, BatchParams *bpc) {
  *slots = p.dedup.slots;
  *n_slots = int64_t(1) << p.dedup.log2cap;
  *st = p.st;
  *hops = s->cfg.hops;
  *bpc = bp;
  args[0] = slots; args[1] = n_slots; args[2] = st; args[3] = hops; args[4] = bpc;
}

static int begin_grid(const Pipe &p) {
  const int64_t n_slots = int64_t(1) << p.dedup.log2cap;
  return (int)std::min<int64_t>(ceil_div(n_slots / 2, 256), 2048);
}

int launch_batch_generate(Server *s, Pipe &p, hipStream_t st, const BatchParams &bp) {
  const int64_t n_slots = int64_t(1) << p.dedup.log2cap;
  hipLaunchKernelGGL(batch_begin_kernel, dim3(begin_grid(p)), dim3(256), 0, st, p.dedup.slots, n_slots, p.st,
                     s->cfg.hops, bp);
  hipLaunchKernelGGL(batch_generate_kernel, dim3((s->cfg.batch_size + 255) / 256), dim3(256), 0, st, s->n_nodes,
                     p.ids, p.labels, p.dedup.slots, p.dedup.log2cap, p.st);
  LMI_HIP(hipGetLastError());
  p.n_seeds = bp.n_seeds;
  p.hops_done = 0;
  return LMI_OK;
}

// Re-points the captured graph's first kernel at this batch's parameters.
int graph_update_begin(Server *s, Pipe &p, const BatchParams &bp) {
  HashSlot *slots; int64_t n_slots; DevState *st; int hops; BatchParams bpc;
  void *args[5];
  begin_args(s, p, bp, args, &slots, &n_slots, &st, &hops, &bpc);
  hipKernelNodeParams kp{};
  kp.func = reinterpret_cast<void *>(batch_begin_kernel);
  kp.gridDim = dim3(begin_grid(p));
  kp.blockDim = dim3(256);
  kp.sharedMemBytes = 0;
  kp.kernelParams = args;
  kp.extra = nullptr;
  LMI_HIP(hipGraphExecKernelNodeSetParams(p.graph_exec, p.begin_node, &kp));
  p.n_seeds = bp.n_seeds;
  p.hops_done = s->cfg.hops;
  return LMI_OK;
}

template <int G>
static void launch_sample_g(Server *s, Pipe &p, hipStream_t st, int hop, int grid) {
  hipLaunchKernelGGL(hop_sample_kernel<G>, dim3(grid), dim3(256), 0, st, p.ids, s->indptr, s->indices,
                     s->n_nodes, s->cfg.fanout[hop], hop, p.st, p.blk_indptr[hop],
                     p.agg_src_ids, p.agg_dst_off, p.dedup.slots, p.dedup.log2cap, p.eslot);
}

int launch_hop(Server *s, Pipe &p, hipStream_t st, int hop) {
  const int f = s->cfg.fanout[hop];
  const int64_t n_max = s->node_cap[hop], e_max = s->edge_cap[hop];
  // 1. per-node counts -> row pointers of the block CSR (= edge placement)
  hipLaunchKernelGGL(hop_count_kernel, dim3(scan_grid(n_max)), dim3(kScanBlock), 0, st, p.ids, s->indptr,
                     s->n_nodes, f, hop, p.st, p.cnt, p.tile_sums);
  LMI_TRY(launch_scan_phases(st, p.cnt, p.blk_indptr[hop], p.tile_sums, &p.st->node_counter[9 + hop],
                             n_max, SCAN_EPI_HOP_EDGES, p.st, hop, &p.st->scan_total));
  // 2. sample + insert
  int G = 4;
  while (G < f) G <<= 1;
  const int grid = (int)std::min<int64_t>(ceil_div(n_max * G, 256), 8192);
  switch (G) {
    case 4: launch_sample_g<4>(s, p, st, hop, grid); break;
    case 8: launch_sample_g<8>(s, p, st, hop, grid); break;
    case 16: launch_sample_g<16>(s, p, st, hop, grid); break;
    case 32: launch_sample_g<32>(s, p, st, hop, grid); break;
    default: launch_sample_g<64>(s, p, st, hop, grid); break;
  }
  // 3. first-occurrence flags -> ranks
  hipLaunchKernelGGL(hop_flag_kernel, dim3(scan_grid(e_max)), dim3(kScanBlock), 0, st, p.dedup.slots,
                     p.eslot, hop, p.st, p.firstv, p.cnt, p.tile_sums);
  LMI_TRY(launch_scan_phases(st, p.cnt, p.rank, p.tile_sums, &p.st->edge_counter[9 + hop + 1], e_max,
                             SCAN_EPI_HOP_NODES, p.st, hop, &p.st->scan_total));
  // 4. relabel
  const int rgrid = (int)std::min<int64_t>(ceil_div(e_max, 256), 4096);
  hipLaunchKernelGGL(hop_relabel_kernel, dim3(rgrid), dim3(256), 0, st, p.firstv, p.rank, p.eslot, hop,
                     p.st, p.agg_src_ids, p.agg_src_off, p.ids, p.dedup.slots);
  LMI_HIP(hipGetLastError());
  p.hops_done = hop + 1;
  return LMI_OK;
}

}  // namespace lmi
