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
//
// A hop is three steps:
//   1. hop_count_sample per-node output counts -> block-CSR row pointers (single-pass
//                       scan), draw positions, write edges, insert sources into the dedup
//                       table; for hop 0 it also stages the seeds.  (Also available as
//                       two kernels, hop_count_scan + hop_sample.)
//   2. hop_flag_scan    first-occurrence flags -> ranks (single-pass scan); first
//                       occurrences append their node to ids[] and publish its local id
//                       in the table; new node count
//   3. fill             local id of every edge source = its table slot's value.  Inside a
//                       batch this rides in extra blocks of the next kernel (the next
//                       hop's step 1, or the cache lookup); hop_fill_kernel does it alone.
#include <algorithm>

#include "scan.hpp"

namespace lmi {

struct HopArgs {
  // graph
  const int64_t *indptr;
  const int32_t *indices;
  int64_t n_nodes;
  int fanout, hop;
  // pipe
  DevState *st;
  int32_t *ids, *labels;
  int32_t *row_ptr;  // block CSR row pointers of this hop
  int32_t *agg_src_ids, *agg_src_off, *agg_dst_off;
  HashSlot *slots;
  int log2cap;
  int32_t *eslot;   // table slot per edge of this hop (| kKnownRepeat)
  ScanChain chain_nodes, chain_edges;
  int max_tiles;
  int stage_seeds;  // hop 0 only: the seeds have not been staged by batch_generate_kernel yet
  int tile_blocks;  // hop_count_sample: blocks [0, tile_blocks) own node tiles, the rest fill
  FillArgs fill;    // the previous hop's last step, carried by hop_count_sample (hop -1: none)
};

// Several mini-batches (pipes) can share every launch of the sampling phase: block b
// works on pipe b mod n (LMI_GRID_ROW).  The kernels are latency-bound, so a second batch
// in the same launch costs far less than a second launch.
constexpr int kMaxGroup = LMI_MAX_GROUP;
struct HopGroup {
  HopArgs p[kMaxGroup];
  int n;
};
struct FillGroup {
  FillArgs p[kMaxGroup];
  int n;
};
struct BeginPipe {
  HashSlot *slots;
  DevState *st;
  ScanChain chain_nodes, chain_edges;
  BatchParams bp;
};
struct BeginGroup {
  BeginPipe p[kMaxGroup];
  int n;
};

// ------------------------------------------------------------ batch start
// Clears the dedup table (key = -1, value = INT_MAX), resets the pipe state and
// the scan chains, and stores the per-batch parameters where later kernels read them.
static __global__ __launch_bounds__(256) void batch_begin_kernel(BeginGroup g, int64_t n_slots, int hops,
                                                                 int max_tiles) {
  LMI_GRID_ROW(g.n);
  HashSlot *slots = g.p[row].slots;
  DevState *st = g.p[row].st;
  const ScanChain chain_nodes = g.p[row].chain_nodes, chain_edges = g.p[row].chain_edges;
  const BatchParams &bp = g.p[row].bp;
  const int64_t tid = (int64_t)bx * blockDim.x + threadIdx.x;
  const int64_t stride = (int64_t)gx * blockDim.x;
  // two slots (16 bytes) per store
  if (bp.clear_table) {
    const int4 fill = make_int4(kEmptyKey, kIntMax, kEmptyKey, kIntMax);
    int4 *p = reinterpret_cast<int4 *>(slots);
    for (int64_t i = tid; i < n_slots / 2; i += stride) p[i] = fill;
  }
  scan_chain_reset(chain_nodes, max_tiles, tid, stride);
  scan_chain_reset(chain_edges, max_tiles, tid, stride);
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
    st->table_tag = bp.table_tag;
    st->table_mask = bp.table_mask;
    st->seeds = bp.seeds;
    st->labels_in = bp.labels;
    st->fault = bp.fault;
  }
}

// Stage the seeds on their own (operator-by-operator use, where the seeds' cache
// lookup runs before the first hop): ids[i] = seed, labels, table[seed] = min(i).
static __global__ __launch_bounds__(256) void batch_generate_kernel(int64_t n_nodes, int32_t *ids, int32_t *labels,
                                                                    HashSlot *slots, int log2cap, DevState *st) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= st->n_seeds) return;
  const int32_t id = st->seeds[i];
  ids[i] = id;
  labels[i] = st->labels_in ? st->labels_in[i] : -1;
  if (id < 0 || id >= n_nodes) {
    raise_fault(st, kFaultBadId);
    return;
  }
  table_insert_min(slots, log2cap, id, i, st->table_tag, st->table_mask);
}

// ------------------------------------------------------------- hop, phase 1
// row_ptr[i] = exclusive prefix of min(deg(ids[i]), fanout) over every node known
// so far; the total is the hop's edge count.  Hop 0 first stages the seeds:
// ids[i] = seed, labels, and table[seed] = min(i) so that a repeated seed resolves
// to its first row.
template <int ITEMS>
static __global__ __launch_bounds__(kScanBlock) void hop_count_scan_kernel(HopGroup g) {
  LMI_GRID_ROW(g.n);
  const HopArgs &a = g.p[row];  // this block's pipe (mini-batch)
  constexpr int TILE = kScanBlock * ITEMS;
  __shared__ int lds[kScanBlock / kWave + 1];
  __shared__ int s_prefix;
  DevState *st = a.st;
  const int n = st->node_counter[9 + a.hop];
  const int n_tiles = (n + TILE - 1) / TILE;
  if (n_tiles == 0) {
    if (bx == 0 && threadIdx.x == 0) {
      a.row_ptr[0] = 0;
      scan_epilogue(SCAN_EPI_HOP_EDGES, st, a.hop, 0);
    }
    return;
  }
  const int tile = bx;
  if (tile < n_tiles) {
    const int base = tile * TILE + threadIdx.x * ITEMS;
    int32_t id[ITEMS];
    // 1. node ids (hop 0: stage the seeds)
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int i = base + j;
      id[j] = -1;
      if (i < n) {
        if (a.stage_seeds) {
          id[j] = st->seeds[i];
          a.ids[i] = id[j];
          a.labels[i] = st->labels_in ? st->labels_in[i] : -1;
        } else {
          id[j] = a.ids[i];
        }
        if (id[j] < 0 || id[j] >= a.n_nodes) {
          if (a.stage_seeds) raise_fault(st, kFaultBadId);
          id[j] = -1;
        }
      }
    }
    // 2. all row-pointer loads in flight together
    int64_t lo[ITEMS], hi[ITEMS];
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      lo[j] = hi[j] = 0;
      if (id[j] >= 0) {
        lo[j] = a.indptr[id[j]];
        hi[j] = a.indptr[id[j] + 1];
      }
    }
    if (a.stage_seeds) {
#pragma unroll
      for (int j = 0; j < ITEMS; ++j)
        if (id[j] >= 0) table_insert_min(a.slots, a.log2cap, id[j], base + j, st->table_tag, st->table_mask);
    }
    int v[ITEMS], sum = 0;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int64_t deg = hi[j] - lo[j];
      v[j] = (int)(deg < (int64_t)a.fanout ? deg : (int64_t)a.fanout);
      sum += v[j];
    }
    int total;
    const int ex = block_exclusive_scan<kScanBlock>(sum, lds, total);
    const int prefix = scan_tile_prefix(a.chain_nodes, tile, total, &s_prefix, st);
    if (prefix == kScanFaultPrefix) return;  // the whole block: no offset, no writes
    int run = prefix + ex;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      if (base + j < n) a.row_ptr[base + j] = run;
      run += v[j];
    }
    if (tile == n_tiles - 1 && threadIdx.x == 0) {
      a.row_ptr[n] = prefix + total;
      scan_epilogue(SCAN_EPI_HOP_EDGES, st, a.hop, prefix + total);
    }
  }
}

// ------------------------------------------------------------- hop, phase 2
// One group of G lanes per node, one lane per output slot.  Rows no longer than
// the fanout are copied whole; longer rows draw `fanout` distinct positions with
// Floyd's rule, the group resolving collisions slot by slot through shuffles.
// Every sampled edge is inserted into the dedup table with candidate value
// n_prev + e (e = edge index inside the hop); atomicMin keeps the first edge.
template <int G>
static __global__ __launch_bounds__(256) void hop_sample_kernel(HopGroup g) {
  LMI_GRID_ROW(g.n);
  const HopArgs &a = g.p[row];  // this block's pipe (mini-batch)
  const DevState *st = a.st;
  const int64_t flat = (int64_t)bx * blockDim.x + threadIdx.x;
  scan_chain_reset(a.chain_edges, a.max_tiles, flat, (int64_t)gx * blockDim.x);
  const uint64_t seed = (uint64_t)st->rng_lo | ((uint64_t)st->rng_hi << 32);
  const int32_t tag = st->table_tag, tag_mask = st->table_mask;
  const int n_prev = st->node_counter[9 + a.hop];
  const int eoff = st->edge_counter[12 + a.hop + 1];
  const int fanout = a.fanout;
  const int lane = threadIdx.x & (G - 1);
  const int group = (int)(flat / G);
  const int n_groups = gx * blockDim.x / G;
  for (int i = group; i < n_prev; i += n_groups) {
    const int32_t v = a.ids[i];
    if (v < 0 || v >= a.n_nodes) continue;
    const int64_t beg = a.indptr[v];
    const int64_t deg = a.indptr[v + 1] - beg;
    const int base = a.row_ptr[i];
    int64_t pick = lane;
    int count;
    if (deg <= (int64_t)fanout) {
      count = (int)deg;
    } else {
      count = fanout;
      const uint32_t j = (uint32_t)(deg - fanout) + (uint32_t)lane;
      uint32_t t = 0xFFFFFFFFu;
      if (lane < fanout) t = __umulhi(sample_draw(seed, (uint32_t)a.hop, (uint32_t)v, (uint32_t)lane), j + 1u);
      bool dup = false;
      for (int q = 0; q + 1 < fanout; ++q) {
        const uint32_t mine = dup ? j : t;
        const uint32_t p = __shfl(mine, q, G);
        if (lane > q && t == p) dup = true;
      }
      pick = dup ? j : t;
    }
    if (lane < count) {
      const int32_t nbr = a.indices[beg + pick];
      const int e = base + lane;
      a.agg_src_ids[eoff + e] = nbr;
      a.agg_dst_off[eoff + e] = i;
      a.eslot[e] = (int)table_insert_min(a.slots, a.log2cap, nbr, n_prev + e, tag, tag_mask);
    }
  }
}

// Variant with LDS-staged probes: the (up to 256) edges a block draws in one step are
// first deduplicated in a 512-entry LDS hash table; only the lowest edge of each
// distinct neighbour probes the HBM table, the other lanes copy its slot.  Same
// results (the HBM table still sees the minimum edge index per key).
template <int G>
static __global__ __launch_bounds__(256) void hop_sample_lds_kernel(HopGroup g) {
  LMI_GRID_ROW(g.n);
  const HopArgs &a = g.p[row];  // this block's pipe (mini-batch)
  constexpr int TAB = 512;
  __shared__ int32_t lds_key[TAB];
  __shared__ int32_t lds_min[TAB];
  __shared__ int32_t lds_slot[TAB];
  const DevState *st = a.st;
  const int64_t flat = (int64_t)bx * blockDim.x + threadIdx.x;
  scan_chain_reset(a.chain_edges, a.max_tiles, flat, (int64_t)gx * blockDim.x);
  const uint64_t seed = (uint64_t)st->rng_lo | ((uint64_t)st->rng_hi << 32);
  const int n_prev = st->node_counter[9 + a.hop];
  const int eoff = st->edge_counter[12 + a.hop + 1];
  const int fanout = a.fanout;
  const int lane = threadIdx.x & (G - 1);
  const int group = (int)(flat / G);
  const int n_groups = gx * blockDim.x / G;
  const int groups_per_block = 256 / G;
  // uniform trip count per block: the block's first group decides
  for (int i0 = bx * groups_per_block; i0 < n_prev; i0 += n_groups) {
    const int i = i0 + (group - bx * groups_per_block);
    for (int t = threadIdx.x; t < TAB; t += 256) {
      lds_key[t] = kEmptyKey;
      lds_min[t] = kIntMax;
    }
    __syncthreads();
    bool active = false;
    int32_t nbr = -1;
    int e = 0, h = 0;
    if (i < n_prev) {
      const int32_t v = a.ids[i];
      if (v >= 0 && v < a.n_nodes) {
        const int64_t beg = a.indptr[v];
        const int64_t deg = a.indptr[v + 1] - beg;
        const int base = a.row_ptr[i];
        int64_t pick = lane;
        int count;
        if (deg <= (int64_t)fanout) {
          count = (int)deg;
        } else {
          count = fanout;
          const uint32_t j = (uint32_t)(deg - fanout) + (uint32_t)lane;
          uint32_t t = 0xFFFFFFFFu;
          if (lane < fanout) t = __umulhi(sample_draw(seed, (uint32_t)a.hop, (uint32_t)v, (uint32_t)lane), j + 1u);
          bool dup = false;
          for (int q = 0; q + 1 < fanout; ++q) {
            const uint32_t mine = dup ? j : t;
            const uint32_t p = __shfl(mine, q, G);
            if (lane > q && t == p) dup = true;
          }
          pick = dup ? j : t;
        }
        if (lane < count) {
          active = true;
          nbr = a.indices[beg + pick];
          e = base + lane;
          a.agg_src_ids[eoff + e] = nbr;
          a.agg_dst_off[eoff + e] = i;
          h = (int)(((uint32_t)nbr * 0x9E3779B1u) >> 23);  // 9 bits
          while (true) {
            const int32_t k = atomicCAS(&lds_key[h], kEmptyKey, nbr);
            if (k == kEmptyKey || k == nbr) break;
            h = (h + 1) & (TAB - 1);
          }
          atomicMin(&lds_min[h], e);
        }
      }
    }
    __syncthreads();
    if (active && lds_min[h] == e)
      lds_slot[h] = (int)table_insert_min(a.slots, a.log2cap, nbr, n_prev + e, st->table_tag, st->table_mask);
    __syncthreads();
    // an edge that lost inside the block is a repeat whatever the table said to the winner
    if (active) a.eslot[e] = (lds_min[h] == e) ? lds_slot[h] : (lds_slot[h] | (int32_t)kKnownRepeat);
    __syncthreads();
  }
}

// ------------------------------------------------- hop, phases 1 and 2 in one launch
// One tile of NPB nodes per block.  Wavefront 0 loads the tile's row pointers, scans
// min(deg, fanout) across its lanes and obtains the tile's edge offset by look-back
// over the earlier tiles; then the whole block samples the tile's nodes, G lanes per
// node, from the row bounds kept in LDS.  Same outputs as hop_count_scan_kernel
// followed by hop_sample_kernel, one launch and one row-pointer read less.
template <int G, int NPB>
static __global__ __launch_bounds__(256) void hop_count_sample_kernel(HopGroup g) {
  LMI_GRID_ROW(g.n);
  const HopArgs &a = g.p[row];  // this block's pipe (mini-batch)
  static_assert(NPB <= kWave && NPB >= 256 / G, "tile = one wavefront of nodes at most, one pass at least");
  __shared__ int32_t s_id[NPB];
  __shared__ int64_t s_beg[NPB], s_deg[NPB];
  __shared__ int s_row[NPB];
  __shared__ int s_prefix;
  DevState *st = a.st;
  const int64_t flat = (int64_t)bx * blockDim.x + threadIdx.x;
  scan_chain_reset(a.chain_edges, a.max_tiles, flat, (int64_t)gx * blockDim.x);
  if (bx >= a.tile_blocks) {  // extra blocks: the previous hop's local ids
    fill_local_ids(a.fill, (int64_t)(bx - a.tile_blocks) * blockDim.x + threadIdx.x,
                   (int64_t)(gx - a.tile_blocks) * blockDim.x);
    return;
  }
  const int n_prev = st->node_counter[9 + a.hop];
  const int n_tiles = (n_prev + NPB - 1) / NPB;
  if (n_tiles == 0) {
    if (bx == 0 && threadIdx.x == 0) {
      a.row_ptr[0] = 0;
      scan_epilogue(SCAN_EPI_HOP_EDGES, st, a.hop, 0);
    }
    return;
  }
  const int tile = bx;
  if (tile >= n_tiles) return;
  // ---- counts, tile scan (wavefront 0)
  const int t = threadIdx.x;
  const int my = tile * NPB + t;
  int cnt = 0, ex = 0, total = 0;
  int32_t id = -1;
  int64_t lo = 0, hi = 0;
  if (t < kWave) {
    if (t < NPB && my < n_prev) {
      if (a.stage_seeds) {
        id = st->seeds[my];
        a.ids[my] = id;
        a.labels[my] = st->labels_in ? st->labels_in[my] : -1;
      } else {
        id = a.ids[my];
      }
      if (id < 0 || id >= a.n_nodes) {
        if (a.stage_seeds) raise_fault(st, kFaultBadId);
        id = -1;
      }
    }
    if (id >= 0) {
      lo = a.indptr[id];
      hi = a.indptr[id + 1];
      if (a.stage_seeds) table_insert_min(a.slots, a.log2cap, id, my, st->table_tag, st->table_mask);
    }
    const int64_t deg = hi - lo;
    cnt = (int)(deg < (int64_t)a.fanout ? deg : (int64_t)a.fanout);
    const int inc = wave_inclusive_scan(cnt);
    ex = inc - cnt;
    total = __shfl(inc, kWave - 1, kWave);
  }
  const int prefix = scan_tile_prefix(a.chain_nodes, tile, total, &s_prefix, st);
  if (prefix == kScanFaultPrefix) return;  // the whole block: no offset, no writes
  if (t < NPB) {
    s_id[t] = id;
    s_beg[t] = lo;
    s_deg[t] = hi - lo;
    s_row[t] = prefix + ex;
    if (my < n_prev) a.row_ptr[my] = prefix + ex;
  }
  if (tile == n_tiles - 1 && t == 0) {
    a.row_ptr[n_prev] = prefix + total;
    scan_epilogue(SCAN_EPI_HOP_EDGES, st, a.hop, prefix + total);
  }
  __syncthreads();
  // ---- sampling: the edge offset of the hop is fixed by the hops before it
  const uint64_t seed = (uint64_t)st->rng_lo | ((uint64_t)st->rng_hi << 32);
  const int32_t tag = st->table_tag, tag_mask = st->table_mask;
  const int eoff = (a.hop == 0) ? 0 : st->edge_counter[12 + a.hop] + st->edge_counter[9 + a.hop];
  const int fanout = a.fanout;
  const int lane = t & (G - 1);
  for (int q = t / G; q < NPB; q += 256 / G) {
    const int i = tile * NPB + q;
    if (i >= n_prev) break;
    const int32_t v = s_id[q];
    if (v < 0) continue;
    const int64_t beg = s_beg[q], deg = s_deg[q];
    const int base = s_row[q];
    int64_t pick = lane;
    int count;
    if (deg <= (int64_t)fanout) {
      count = (int)deg;
    } else {
      count = fanout;
      const uint32_t j = (uint32_t)(deg - fanout) + (uint32_t)lane;
      uint32_t d = 0xFFFFFFFFu;
      if (lane < fanout) d = __umulhi(sample_draw(seed, (uint32_t)a.hop, (uint32_t)v, (uint32_t)lane), j + 1u);
      bool dup = false;
      for (int r = 0; r + 1 < fanout; ++r) {
        const uint32_t mine = dup ? j : d;
        const uint32_t p = __shfl(mine, r, G);
        if (lane > r && d == p) dup = true;
      }
      pick = dup ? j : d;
    }
    if (lane < count) {
      const int32_t nbr = a.indices[beg + pick];
      const int e = base + lane;
      a.agg_src_ids[eoff + e] = nbr;
      a.agg_dst_off[eoff + e] = i;
      a.eslot[e] = (int)table_insert_min(a.slots, a.log2cap, nbr, n_prev + e, tag, tag_mask);
    }
  }
}

// ------------------------------------------------------------- hop, step 2
// An edge is the first occurrence of a new node iff the table value of its source names
// the edge itself (n_prev + e).  Its rank among first occurrences (single-pass scan) is the
// node's place after the n_prev known nodes: the edge appends the node to ids[] and
// publishes the local id in the table.  Publishing while other tiles still read is safe: a
// later edge of the same node compares the value with its own, larger, index either way.
template <int ITEMS>
static __global__ __launch_bounds__(kScanBlock) void hop_flag_scan_kernel(HopGroup g) {
  LMI_GRID_ROW(g.n);
  const HopArgs &a = g.p[row];  // this block's pipe (mini-batch)
  constexpr int TILE = kScanBlock * ITEMS;
  __shared__ int lds[kScanBlock / kWave + 1];
  __shared__ int s_prefix;
  DevState *st = a.st;
  const int64_t flat = (int64_t)bx * blockDim.x + threadIdx.x;
  scan_chain_reset(a.chain_nodes, a.max_tiles, flat, (int64_t)gx * blockDim.x);  // for the next hop
  const int n_prev = st->node_counter[9 + a.hop];
  const int n = st->edge_counter[9 + a.hop + 1];
  const int eoff = st->edge_counter[12 + a.hop + 1];
  const int n_tiles = (n + TILE - 1) / TILE;
  if (n_tiles == 0) {
    if (bx == 0 && threadIdx.x == 0) scan_epilogue(SCAN_EPI_HOP_NODES, st, a.hop, 0);
    return;
  }
  const int tile = bx;
  if (tile < n_tiles) {
    const int base = tile * TILE + threadIdx.x * ITEMS;
    int v[ITEMS], slot[ITEMS], sum = 0;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      const int e = base + j;
      int flag = 0;
      slot[j] = 0;
      if (e < n) {
        const int32_t es = a.eslot[e];  // sign bit = kKnownRepeat: no need to look
        slot[j] = es & (int32_t)~kKnownRepeat;
        if (es >= 0) flag = (a.slots[slot[j]].val == n_prev + e) ? 1 : 0;
      }
      v[j] = flag;
      sum += flag;
    }
    int total;
    const int ex = block_exclusive_scan<kScanBlock>(sum, lds, total);
    const int prefix = scan_tile_prefix(a.chain_edges, tile, total, &s_prefix, st);
    if (prefix == kScanFaultPrefix) return;  // the whole block: no ranks, no writes
    int run = prefix + ex;
#pragma unroll
    for (int j = 0; j < ITEMS; ++j) {
      if (v[j]) {
        const int local = n_prev + run;
        a.ids[local] = a.agg_src_ids[eoff + base + j];
        a.slots[slot[j]].val = local;
      }
      run += v[j];
    }
    if (tile == n_tiles - 1 && threadIdx.x == 0) scan_epilogue(SCAN_EPI_HOP_NODES, st, a.hop, prefix + total);
  }
}

// ------------------------------------------------------------- hop, step 3
static __global__ __launch_bounds__(256) void hop_fill_kernel(FillGroup g) {
  LMI_GRID_ROW(g.n);
  const FillArgs &f = g.p[row];
  fill_local_ids(f, (int64_t)bx * blockDim.x + threadIdx.x, (int64_t)gx * blockDim.x);
}

// ---------------------------------------------------------------- launchers
static ScanChain chain_of(const Pipe &p, int which) { return ScanChain{p.chain_status[which]}; }

static int begin_grid(const Pipe &p) {
  const int64_t n_slots = int64_t(1) << p.dedup.log2cap;
  return (int)std::min<int64_t>(ceil_div(n_slots / 2, 256), 2048);
}

static BeginGroup begin_group(Pipe *const *pp, const BatchParams *bps, int n) {
  BeginGroup g{};
  g.n = n;
  for (int k = 0; k < n; ++k) {
    g.p[k].slots = pp[k]->dedup.slots;
    g.p[k].st = pp[k]->st;
    g.p[k].chain_nodes = chain_of(*pp[k], 0);
    g.p[k].chain_edges = chain_of(*pp[k], 1);
    g.p[k].bp = bps[k];
  }
  return g;
}

// First kernel of a batch for each of the n pipes (one launch); stage_seeds also stages the
// seeds in a kernel of their own (operator-by-operator use, one pipe).
int launch_batch_generate(Server *s, Pipe *const *pp, const BatchParams *bps, int n, hipStream_t st, bool stage_seeds) {
  Pipe &p0 = *pp[0];
  const int64_t n_slots = int64_t(1) << p0.dedup.log2cap;
  hipLaunchKernelGGL(batch_begin_kernel, dim3((begin_grid(p0)) * n), dim3(256), 0, st, begin_group(pp, bps, n), n_slots,
                     s->cfg.hops, p0.max_tiles);
  if (stage_seeds)
    for (int k = 0; k < n; ++k)
      hipLaunchKernelGGL(batch_generate_kernel, dim3((s->cfg.batch_size + 255) / 256), dim3(256), 0, st, s->n_nodes,
                         pp[k]->ids, pp[k]->labels, pp[k]->dedup.slots, pp[k]->dedup.log2cap, pp[k]->st);
  LMI_HIP(hipGetLastError());
  for (int k = 0; k < n; ++k) {
    pp[k]->n_seeds = bps[k].n_seeds;
    pp[k]->hops_done = 0;
  }
  return LMI_OK;
}

// Re-points the captured graph's first kernel at this batch's parameters.
int graph_update_begin(Server *s, Pipe &p, const BatchParams &bp) {
  Pipe *pp[1] = {&p};
  BeginGroup g = begin_group(pp, &bp, 1);
  int64_t n_slots = int64_t(1) << p.dedup.log2cap;
  int hops = s->cfg.hops;
  int max_tiles = p.max_tiles;
  void *args[4] = {&g, &n_slots, &hops, &max_tiles};
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

// One hop for each of the n pipes, all in the same launches (the pipes are in step: same hop,
// same pending fill).
int launch_hop(Server *s, Pipe *const *pp, int n, hipStream_t st, int hop, bool stage_seeds, bool defer_fill) {
  const int f = s->cfg.fanout[hop];
  const int64_t n_max = s->node_cap[hop], e_max = s->edge_cap[hop];
  Pipe &p0 = *pp[0];
  HopGroup g{};
  g.n = n;
  for (int k = 0; k < n; ++k) {
    Pipe &p = *pp[k];
    HopArgs &a = g.p[k];
    a.indptr = s->indptr;
    a.indices = s->indices;
    a.n_nodes = s->n_nodes;
    a.fanout = f;
    a.hop = hop;
    a.st = p.st;
    a.ids = p.ids;
    a.labels = p.labels;
    a.row_ptr = p.blk_indptr[hop];
    a.agg_src_ids = p.agg_src_ids;
    a.agg_src_off = p.agg_src_off;
    a.agg_dst_off = p.agg_dst_off;
    a.slots = p.dedup.slots;
    a.log2cap = p.dedup.log2cap;
    a.eslot = p.eslot[hop & 1];
    a.chain_nodes = chain_of(p, 0);
    a.chain_edges = chain_of(p, 1);
    a.max_tiles = p.max_tiles;
    a.stage_seeds = (hop == 0 && stage_seeds) ? 1 : 0;
    a.fill.hop = -1;
  }
  int G = 4;
  while (G < f) G <<= 1;
  const bool fused = s->fuse_count && !s->lds_dedup;
  if (!fused) LMI_TRY(launch_fill(s, pp, n, st));
  if (fused) {
    // counts, scan and sampling in one launch, one tile of nodes per block; a hop left
    // pending gets its local ids filled in by extra blocks behind the tile blocks
    const int npb = hop_tile_nodes(n_max, G, s->fuse_small_max);
    const int tile_blocks = (int)ceil_div(std::max<int64_t>(n_max, 1), npb);
    int grid = tile_blocks;
    if (p0.fill_pending >= 0) grid += fill_blocks(s->edge_cap[p0.fill_pending], 256);
    for (int k = 0; k < n; ++k) {
      g.p[k].tile_blocks = tile_blocks;
      if (pp[k]->fill_pending >= 0) g.p[k].fill = fill_args(*pp[k], pp[k]->fill_pending);
      pp[k]->fill_pending = -1;
    }
#define LMI_FUSED(GG)                                                                                   \
  if (npb == 64)                                                                                        \
    hipLaunchKernelGGL((hop_count_sample_kernel<GG, 64>), dim3((grid) * n), dim3(256), 0, st, g);          \
  else                                                                                                  \
    hipLaunchKernelGGL((hop_count_sample_kernel<GG, (256 / GG)>), dim3((grid) * n), dim3(256), 0, st, g);
    switch (G) {
      case 4: LMI_FUSED(4) break;
      case 8: LMI_FUSED(8) break;
      case 16: LMI_FUSED(16) break;
      case 32: LMI_FUSED(32) break;
      default: LMI_FUSED(64) break;
    }
#undef LMI_FUSED
  } else {
    // one tile per block (blocks past the real item count leave at once); few items per
    // thread while that keeps the tile count near a thousand: the row-pointer reads are
    // dependent random accesses, so parallelism matters more than per-thread work
    const int64_t nm = std::max<int64_t>(n_max, 1);
    if (nm <= 256 * 1024)
      hipLaunchKernelGGL(hop_count_scan_kernel<1>, dim3(((int)ceil_div(nm, kScanBlock)) * n), dim3(kScanBlock), 0, st, g);
    else if (nm <= 512 * 1024)
      hipLaunchKernelGGL(hop_count_scan_kernel<2>, dim3(((int)ceil_div(nm, kScanBlock * 2)) * n), dim3(kScanBlock), 0, st, g);
    else if (nm <= 1024 * 1024)
      hipLaunchKernelGGL(hop_count_scan_kernel<4>, dim3(((int)ceil_div(nm, kScanBlock * 4)) * n), dim3(kScanBlock), 0, st, g);
    else
      hipLaunchKernelGGL(hop_count_scan_kernel<8>, dim3(((int)ceil_div(nm, kScanBlock * 8)) * n), dim3(kScanBlock), 0, st, g);
    const int grid = (int)std::min<int64_t>(ceil_div(n_max * G, 256), 8192);
    if (s->lds_dedup) {
      switch (G) {
        case 4: hipLaunchKernelGGL(hop_sample_lds_kernel<4>, dim3((grid) * n), dim3(256), 0, st, g); break;
        case 8: hipLaunchKernelGGL(hop_sample_lds_kernel<8>, dim3((grid) * n), dim3(256), 0, st, g); break;
        case 16: hipLaunchKernelGGL(hop_sample_lds_kernel<16>, dim3((grid) * n), dim3(256), 0, st, g); break;
        case 32: hipLaunchKernelGGL(hop_sample_lds_kernel<32>, dim3((grid) * n), dim3(256), 0, st, g); break;
        default: hipLaunchKernelGGL(hop_sample_lds_kernel<64>, dim3((grid) * n), dim3(256), 0, st, g); break;
      }
    } else {
      switch (G) {
        case 4: hipLaunchKernelGGL(hop_sample_kernel<4>, dim3((grid) * n), dim3(256), 0, st, g); break;
        case 8: hipLaunchKernelGGL(hop_sample_kernel<8>, dim3((grid) * n), dim3(256), 0, st, g); break;
        case 16: hipLaunchKernelGGL(hop_sample_kernel<16>, dim3((grid) * n), dim3(256), 0, st, g); break;
        case 32: hipLaunchKernelGGL(hop_sample_kernel<32>, dim3((grid) * n), dim3(256), 0, st, g); break;
        default: hipLaunchKernelGGL(hop_sample_kernel<64>, dim3((grid) * n), dim3(256), 0, st, g); break;
      }
    }
  }
  const int64_t em = std::max<int64_t>(e_max, 1);
  if (em <= 1024 * 1024)
    hipLaunchKernelGGL(hop_flag_scan_kernel<2>, dim3(((int)ceil_div(em, kScanBlock * 2)) * n), dim3(kScanBlock), 0, st, g);
  else if (em <= 2560 * 1024)
    hipLaunchKernelGGL(hop_flag_scan_kernel<4>, dim3(((int)ceil_div(em, kScanBlock * 4)) * n), dim3(kScanBlock), 0, st, g);
  else
    hipLaunchKernelGGL(hop_flag_scan_kernel<8>, dim3(((int)ceil_div(em, kScanBlock * 8)) * n), dim3(kScanBlock), 0, st, g);
  LMI_HIP(hipGetLastError());
  for (int k = 0; k < n; ++k) {
    pp[k]->fill_pending = hop;
    pp[k]->hops_done = hop + 1;
  }
  if (!defer_fill) LMI_TRY(launch_fill(s, pp, n, st));
  return LMI_OK;
}

FillArgs fill_args(const Pipe &p, int hop) {
  FillArgs f{};
  f.st = p.st;
  f.slots = p.dedup.slots;
  f.eslot = p.eslot[hop & 1];
  f.agg_src_off = p.agg_src_off;
  f.hop = hop;
  return f;
}

int fill_blocks(int64_t e_max, int block) {  // four edges per thread
  return (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(e_max, (int64_t)block * 4), 1024));
}

int launch_fill(Server *s, Pipe *const *pp, int n, hipStream_t st) {
  const int hop = pp[0]->fill_pending;
  if (hop < 0) return LMI_OK;
  FillGroup g{};
  g.n = n;
  for (int k = 0; k < n; ++k) {
    g.p[k] = fill_args(*pp[k], hop);
    pp[k]->fill_pending = -1;
  }
  hipLaunchKernelGGL(hop_fill_kernel, dim3((fill_blocks(s->edge_cap[hop], 256)) * n), dim3(256), 0, st, g);
  LMI_HIP(hipGetLastError());
  return LMI_OK;
}

}  // namespace lmi
