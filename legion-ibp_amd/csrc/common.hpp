// Shared declarations of the MI355X sampling-server library (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/legion_mi.h"

namespace lmi {

constexpr int kWave = 64;
constexpr int32_t kEmptyKey = -1;
constexpr int32_t kUntaggedMask = (int32_t)0x80000000u;  // tag mask of an untagged table: only key -1 is free
constexpr int32_t kIntMax = 0x7fffffff;

// ---------------------------------------------------------------- errors
void set_error(const char *fmt, ...);
#define LMI_HIP(call)                                                                    \
  do {                                                                                   \
    hipError_t e_ = (call);                                                              \
    if (e_ != hipSuccess) {                                                              \
      lmi::set_error("%s failed: %s (%s:%d)", #call, hipGetErrorString(e_), __FILE__,    \
                     __LINE__);                                                          \
      (void)hipGetLastError(); /* reported here: a later launch check must not see it */ \
      return LMI_ERR_HIP;                                                                \
    }                                                                                    \
  } while (0)
#define LMI_TRY(call)            \
  do {                           \
    int rc_ = (call);            \
    if (rc_ != LMI_OK) return rc_; \
  } while (0)
#define LMI_FAIL(code, ...)        \
  do {                             \
    lmi::set_error(__VA_ARGS__);   \
    return (code);                 \
  } while (0)

// ------------------------------------------------------- device-side state
// Lives in HBM, one per pipe.  The two 16-int headers are the reference's
// node_counter / edge_counter (engine/operator_impl.cu:58-91); the rest is
// bookkeeping the kernels read instead of round-tripping through the host.
struct DevState {
  int32_t node_counter[16];
  int32_t edge_counter[16];
  // One miss list per lookup segment (0 = seeds or the whole
  // batch, k = nodes added by hop k); zeroed at batch start.
  int32_t n_miss[LMI_MAX_HOPS + 1];
  int32_t scan_fault;  // a look-back scan gave up waiting (never expected; reported as an error)
  int32_t reserved[LMI_MAX_HOPS];
  int32_t bad_id;      // set when a seed id is outside [0, n_nodes)
  int32_t scan_total;  // total of the last device scan
  // per-batch parameters, written by the first kernel of a batch so that every
  // later kernel (and a replayed HIP graph) reads them from HBM
  uint32_t rng_lo, rng_hi;   // 64-bit Philox key of this batch
  int32_t lru_tick;
  int32_t n_seeds;
  int32_t table_tag, table_mask;  // epoch tag of this batch's dedup-table keys (table_insert_min)
  const int32_t *seeds;      // device address of this batch's seed ids
  const int32_t *labels_in;  // device address of their labels (or null)
  int32_t *fault;            // the server's sticky fault words in pinned host memory (raise_fault), or null
};

enum { kFaultBadId = 0, kFaultScan = 1 };  // index of a condition in the server's sticky fault words

struct HashSlot {  // 8-byte open-addressing slot: one 64-bit load per probe
  int32_t key;
  int32_t val;
};

struct Table {  // id -> value, linear probing, capacity = 2^log2cap
  HashSlot *slots = nullptr;
  int32_t log2cap = 0;
  __host__ __device__ uint32_t mask() const { return (1u << log2cap) - 1u; }
  size_t bytes() const { return slots ? (size_t(8) << log2cap) : 0; }
};

struct Pipe {
  // outputs (reference: per-pipe MemoryPool / IPC buffers)
  int32_t *ids = nullptr;
  void *features = nullptr;
  int32_t *labels = nullptr;
  int32_t *agg_src_ids = nullptr, *agg_src_off = nullptr, *agg_dst_off = nullptr;
  int32_t *blk_indptr[LMI_MAX_HOPS] = {nullptr, nullptr, nullptr};
  int32_t *cache_index = nullptr;
  DevState *st = nullptr;
  // scratch
  Table dedup;                 // global id -> local id (per batch)
  int32_t *eslot[2] = {nullptr, nullptr};  // [max_edges_hop] table slot of each edge's source; hops alternate
                                           // so that a hop's slots survive into the next hop's first kernel
  int32_t epoch = 0;           // dedup-table epoch of the last batch
  int id_bits = 0;             // key bits below the epoch tag when that batch ran
  bool table_dirty = true;     // the table must be wiped before its next use
  int fill_pending = -1;       // hop whose edge sources still wait for their local ids (launch_fill)
  unsigned long long *chain_status[2] = {nullptr, nullptr};  // look-back scan state: [0] node scans, [1] edge scans
  int32_t max_tiles = 0;
  int2 *miss_list = nullptr;   // [max_nodes] (row, id) pairs of cache misses
  int32_t *lru_fill = nullptr;                        // [max_nodes] slot granted to a miss
  int32_t *lru_next = nullptr;                        // [max_nodes] next row in the list of misses of the same LRU set
  hipEvent_t fork = nullptr, join = nullptr;
  hipEvent_t fork_early = nullptr;  // releases the side stream for the first hops' misses while later hops are still sampled
  // The event that marks the end of this pipe's side-stream work: its own `join`, or that of the
  // first pipe of the group its misses were gathered with (one record and one wait per group: a
  // wait on another queue's event costs a stream about 10 us, fired or not).
  hipEvent_t join_of = nullptr;
  bool side_pending = false;   // the side stream may still owe this pipe's miss rows (join_of not yet seen complete)
  bool join_waited = false;    // a wait for join_of has been queued on join_waiter: that stream needs no second one,
  hipStream_t join_waiter = nullptr;  // any other stream still does
  // The caller's stream that carried the pipe's last batch, and whether that stream still holds work
  // of the batch that `join_of` does not cover (everything when no side stream is used; the HBM
  // gather when the side stream was released ahead of it).  A later call that uses the pipe from
  // ANOTHER stream is then ordered behind `last_stream` through `handover` (pipe_join).
  hipStream_t last_stream = nullptr;
  bool tail_unjoined = false;
  hipEvent_t handover = nullptr;
  int32_t *seed_stage = nullptr;  // [batch_size] host seeds land here
  int32_t n_seeds = 0;
  int32_t hops_done = 0;
  // HIP graph of one whole batch minus the feature gather (captured on first use)
  hipGraphExec_t graph_exec = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphNode_t begin_node = nullptr;
};

// per-batch scalars, the only arguments that change between graph replays
struct BatchParams {
  int32_t n_seeds;
  int32_t lru_tick;
  int32_t table_tag, table_mask;  // see table_insert_min
  int32_t clear_table;            // 1: the epochs ran out (or the table is new): wipe it first
  int32_t pad;
  uint64_t rng_seed;
  const int32_t *seeds;
  const int32_t *labels;
  int32_t *fault;  // device-visible address of the server's sticky fault words
};

struct EventPair {  // device time between two recorded events, attributed to `kind`
  hipEvent_t a, b;
  int kind;
};

struct Server {
  lmi_config cfg{};
  int64_t max_nodes = 0, max_edges = 0, max_edges_hop = 0;
  int64_t node_cap[LMI_MAX_HOPS + 1] = {0, 0, 0, 0};  // worst-case n_k
  int64_t edge_cap[LMI_MAX_HOPS] = {0, 0, 0};         // worst-case e_k
  int64_t row_bytes = 0;
  // storage
  const int64_t *indptr = nullptr;
  const int32_t *indices = nullptr;
  int64_t n_nodes = 0, n_edges = 0;
  bool own_graph = false;
  const uint8_t *feat = nullptr;  // device-visible address of the feature table
  int64_t feat_rows = 0;
  int feat_loc = LMI_LOC_HOST;
  int32_t *set_ids[3] = {nullptr, nullptr, nullptr};
  int32_t *set_labels[3] = {nullptr, nullptr, nullptr};
  int64_t set_n[3] = {0, 0, 0};
  int32_t set_batch[3] = {0, 0, 0};  // ids per sliced batch; 0 = cfg.batch_size
  // cache
  int policy = LMI_POLICY_DEGREE;    // ranking key of the static / int8 hot set
  uint32_t *hot = nullptr;           // [n_nodes] presampling appearance counts
  int cache_kind = LMI_CACHE_NONE;
  int table_kind = LMI_TABLE_HASH;
  int64_t cache_rows = 0;
  int64_t cache_row_bytes = 0;
  uint8_t *cache_data = nullptr;     // [cache_rows][cache_row_bytes]
  float *cache_scale = nullptr;      // int8: per-row scale
  Table id_table;                    // hash id -> slot
  int32_t *slot_of = nullptr;        // direct id -> slot
  uint4 *rank_tab = nullptr;         // per 64 ids: {bits lo, bits hi, rank of first id, 0}
  int64_t lru_sets = 0;
  int32_t lru_ways = 0;
  int32_t lru_tick = 0;
  int32_t *lru_keys = nullptr, *lru_use = nullptr;  // one array of per-set records: `ways` keys, then `ways` ticks;
                                                    // way w of set s: lru_keys[(s * 2) * ways + w], lru_use[same]
  int32_t *lru_head = nullptr;  // [sets] first row of the set's list of misses while a batch is inserted, else -1
  hipEvent_t side_idle = nullptr;  // recorded behind the last host-link gather issued on the side stream
  bool side_busy = false;
  int protect_hits = 0;            // 1: HBM gathers wait until earlier host-link gathers have drained
  int miss_blocks_early = 0;       // grid of the host-link gather released by split_lookup (0 = miss_blocks)
  int split_lookup = 0;            // 1 (always) or 2 (groups of more than one batch): the seeds and the first hop's
                                   // nodes are looked up before the later hops are sampled and their misses start
                                   // over the host link then (static / int8 cache, 2+ hops); 0: one lookup at the end
  int early_fork = 2;              // when the side stream is released ahead of the HBM gather instead of behind it:
                                   // 0 never, 1 always, 2 for groups of batches (their host-link gather then starts a
                                   // whole HBM gather earlier, which is what a short run or a first batch waits for)
  int lru_early_miss = 1;          // 1: with the LRU cache the host-link gather starts beside the HBM gather
  int group_miss = 1;              // 1: the host-link gathers of a group of batches are one launch
  hipEvent_t lru_ready = nullptr;  // recorded when an LRU insertion has settled keys and ticks: the next lookup waits for it
  bool lru_pending = false;        // an insertion may still be running
  hipEvent_t lru_copied = nullptr; // recorded when the granted rows are in the cache: the next HBM gather waits for it
  bool lru_copy_pending = false;
  // sticky fault words in pinned + mapped host memory, written by kernels, never cleared by a batch:
  // [0] a seed id outside [0, n_nodes), [1] a look-back scan gave up
  volatile int32_t *fault_host = nullptr;
  int32_t *fault_dev = nullptr;  // the same words as the device addresses them
  bool fault_told[2] = {false, false};  // lmi_batch_wait has reported the condition once already
  // row counts the gather kernels leave behind, one word per pipe of a launch, in the same pinned allocation
  volatile int32_t *rows_seen_host = nullptr;
  int32_t *rows_seen_dev = nullptr;
  // pipes
  std::vector<Pipe> pipes;
  hipStream_t side = nullptr;  // server-owned second stream for gathers that must not hold up the caller's stream
  // tuning
  int gather_lpr = 0;     // lanes per row (0 = auto)
  int gather_vec = 0;     // bytes per lane access (0 = widest that fits: 16)
  int gather_unroll = 0;  // rows (units) in flight per lane; 0 = the mover's own best: 1 for the lane-group mover
                          // (a few percent ahead of 4), 2 for the flat gather and the tiled movers
  int gather_tile_rows = 0;  // tiled movers: rows per tile; 0 = the mover's own rule: about 8 KB worth of rows,
                             // 2..64 (256 for rows under 128 bytes); the tiled int8 gather takes 32
  int gather_blocks = 0;  // blocks per pipe; 0 = auto (auto_gather_blocks)
  int gather_nt = 1;      // non-temporal output stores
  int gather_adaptive = 1;   // gather grids sized by the row counts of recent launches instead of the worst case
  int gather_flat = 0;    // HBM gather of hits: 0 / 3 the flat gather (gather_rows_flat_kernel); 1 the LDS-tiled
                          // mover; 2 power-of-two lane groups, tiled only when no lane group fits the row
  int miss_flat = 0;      // the same choice for the host-link gather
  int int8_epl = 0;       // tiled int8 gather: elements per lane (0 = one 16-byte store per lane: 8 fp16 or 4 fp32)
  int64_t fuse_small_max = 32768;  // hops of at most this many nodes use the small tile of hop_tile_nodes
  int64_t table_epochs = int64_t(1) << 30;  // batches a dedup table serves between wipes, less one (also
                                            // bounded by the key bits the node ids leave free)
  int fuse_count = 1;     // 1: row counts, their scan and the sampling of a hop share one launch
  int lds_dedup = 0;      // 1: hop_sample stages its probes through an LDS hash table
  int split_miss = 1;     // gather schedule, see launch_gather_group
  int use_graph = 0;      // 1: lmi_run_once replays a captured HIP graph of the sampling kernels (measured
                          // 2-3 % slower than plain launches here: the host enqueues a batch in 85 us,
                          // well inside its 205 us of device time, and a graph's end costs 9 us)
  int miss_blocks = 32;   // grid of the host-link gather: enough reads in flight to fill the link, few enough
                          // not to crowd HBM traffic out of the memory pipeline
  int miss_unroll = 1;    // rows in flight per lane in the host-link gather
  // profiling
  bool prof_on = false;                 // the batch being issued is profiled (events + device row counters)
  int prof_level = 0;                   // 0 off, 1 every phase bracketed, 2 only the gather kernels
  int prof_every = 1;                   // profile one batch in this many (tuning key "profile_every")
  int64_t prof_seq = 0;                 // batches begun since profiling was switched on
  std::vector<EventPair> prof_events;   // recorded, not yet resolved
  std::vector<hipEvent_t> prof_used;    // every event recorded since the last read (pairs may share one)
  std::vector<hipEvent_t> prof_free;    // recycled events
  int prof_open = -1;                   // pair still waiting for its end event on the caller's stream
  unsigned long long *d_prof_rows = nullptr;  // device counters: [0] rows offered to hit gathers, [1] miss rows
  lmi_profile prof{};
  int32_t *d_scalar = nullptr;          // small device scratch (counts for build-time launches)
  int n_cu = 256;
};

enum { PROF_GATHER_HIT = 0, PROF_GATHER_MISS = 1, PROF_SAMPLE = 2, PROF_LOOKUP = 3 };

// profiling helpers (api.hip)
// One event closes the pair left open on the caller's stream and opens the next
// phase (next_kind < 0: only close), so a batch costs one event per phase boundary.
hipEvent_t prof_phase(Server *s, hipStream_t st, int *open, int next_kind);
// A start / stop event pair for one kernel launch of kind `kind` (both null when profiling
// is off): handed to hipExtLaunchKernelGGL, which stamps them with the kernel's own begin
// and end, so nothing is queued between the kernel and its neighbours.
void prof_kernel_events(Server *s, int kind, hipEvent_t *start, hipEvent_t *stop);

// sampler.hip
// stage_seeds: also run the seed-staging kernel now (otherwise hop 0 stages them itself)
int launch_batch_generate(Server *s, Pipe *const *pp, const BatchParams *bps, int n, hipStream_t st, bool stage_seeds);
int graph_update_begin(Server *s, Pipe &p, const BatchParams &bp);
// defer_fill: leave the last step of the hop (local ids of the edge sources) to the next
// kernel of the batch -- the next hop's first kernel or the lookup -- which carries it in
// extra blocks; otherwise a kernel of its own finishes the hop.
// The launchers below take n pipes that are in step (same stage of their batches) and serve
// them with the same launches, their blocks interleaved over blockIdx.x (LMI_GRID_ROW).
int launch_hop(Server *s, Pipe *const *pp, int n, hipStream_t st, int hop, bool stage_seeds, bool defer_fill);
int launch_fill(Server *s, Pipe *const *pp, int n, hipStream_t st);  // finishes a hop left pending, if any
struct FillArgs;
FillArgs fill_args(const Pipe &p, int hop);
int fill_blocks(int64_t e_max, int block);  // grid share of a fill over at most e_max edges
int launch_table_clear(Table &t, hipStream_t st);

enum { SCAN_EPI_NONE = 0, SCAN_EPI_HOP_EDGES = 1, SCAN_EPI_HOP_NODES = 2 };

// cache.hip
int cache_build_static(Server *s, int64_t capacity_rows, int table_kind, bool int8);
int cache_build_lru(Server *s, int64_t n_sets, int32_t ways);
void cache_free(Server *s);
// Extra blocks of the lookup finish a hop left pending (launch_hop, defer_fill).  (Finishing
// it on the side stream instead, ahead of the host-link gather, measured 2 % slower.)
int launch_lookup(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg_first, int seg_last);
int launch_hotness(Server *s, Pipe &p, hipStream_t st);
// lru_lists > 0: the LRU insertion of that many miss lists follows the gather on the stream the
// misses were gathered on (the side stream when it is in use), and the caller's stream does not wait.
int launch_gather_seg(Server *s, Pipe &p, hipStream_t st, int seg, int seg_last, int lru_lists);
// The same for n pipes in step: the HBM gathers one after another, one fork, then the
// host-link gathers one after another on the side stream.
// same_stream: hits then misses on `st` whatever the schedule knob says (nothing is left pending).
int launch_gather_group(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg, int seg_last, int lru_lists,
                        bool same_stream = false, int hit_seg_first = -1);
// the host-link gather of segments [seg, seg_last] released now, ahead of the batch's later hops (split_lookup)
int launch_misses_early(Server *s, Pipe *const *pp, int n, hipStream_t st, int seg, int seg_last);
int launch_lru_insert(Server *s, Pipe &p, hipStream_t st, int n_lists);
int lru_wait_ready(Server *s, hipStream_t st);
int lru_wait_copied(Server *s, hipStream_t st);  // orders `st` behind the last LRU insertion
int pipe_join(Pipe &p, hipStream_t st);  // make `st` wait for the pipe's last batch, wherever it ran
int pipe_handover(Pipe &p, hipStream_t st);  // only for what another caller's stream still holds of it
// `st` is about to carry work of the pipe's next batch (after pipe_join)
inline void pipe_begin(Pipe &p, hipStream_t st) {
  p.last_stream = st;
  p.tail_unjoined = true;
}
// the same for n pipes, each distinct event waited on once
int pipes_join(Pipe *const *pp, int n, hipStream_t st);
int cache_dump(Server *s, int32_t *slot_of, int64_t n, int32_t *aux);

inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Nodes per block of the fused count-and-sample kernel for a hop of at most n_max nodes
// sampled G lanes per node: a small hop takes one node per lane group (more, smaller tiles
// keep every CU busy), a large one a full wavefront of nodes.
inline int hop_tile_nodes(int64_t n_max, int G, int64_t small_max = 32768) {
  const int per_pass = 256 / G;
  return (n_max <= small_max && per_pass < 64) ? per_pass : 64;
}

}  // namespace lmi
