// C ABI of the sampling-server hot path (see include/legion_mi.h).
#include <algorithm>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>
#include <type_traits>

#include <hip/hip_ext.h>

#include "common.hpp"

namespace lmi {

static thread_local char g_err[512] = "";

void set_error(const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ------------------------------------------------------------ profiling
static hipEvent_t prof_event(Server *s) {
  if (!s->prof_free.empty()) {
    hipEvent_t e = s->prof_free.back();
    s->prof_free.pop_back();
    return e;
  }
  hipEvent_t e = nullptr;
  (void)hipEventCreate(&e);
  return e;
}

// Ends the open bracket of a stream and starts one of kind `next_kind` (-1: none) with a
// single event record; returns that event, or nullptr when nothing was recorded.  Level 2
// brackets only the gather kernels, so the sampling kernels run back to back as they do
// without profiling.
hipEvent_t prof_phase(Server *s, hipStream_t st, int *open, int next_kind) {
  if (!s->prof_on) {
    *open = -1;
    return nullptr;
  }
  if (s->prof_level == 2 && (next_kind == PROF_SAMPLE || next_kind == PROF_LOOKUP)) next_kind = -1;
  if (*open < 0 && next_kind < 0) return nullptr;
  hipEvent_t e = prof_event(s);
  s->prof_used.push_back(e);
  (void)hipEventRecord(e, st);
  if (*open >= 0) s->prof_events[*open].b = e;
  *open = -1;
  if (next_kind >= 0) {
    s->prof_events.push_back(EventPair{e, nullptr, next_kind});
    *open = (int)s->prof_events.size() - 1;
  }
  return e;
}

// Start of a batch, or of a group of n batches served together: decides whether it is profiled.
static void prof_batch(Server *s, int n = 1) {
  s->prof_on = s->prof_level != 0 && (s->prof_seq++ % std::max(1, s->prof_every)) == 0;
  if (s->prof_on) s->prof.batches += n;
}

void prof_kernel_events(Server *s, int kind, hipEvent_t *start, hipEvent_t *stop) {
  *start = *stop = nullptr;
  if (!s->prof_on) return;
  EventPair p{prof_event(s), prof_event(s), kind};
  s->prof_used.push_back(p.a);
  s->prof_used.push_back(p.b);
  s->prof_events.push_back(p);
  *start = p.a;
  *stop = p.b;
}

// The captured batch graphs hold the graph, cache-table and tuning state by value:
// anything that changes those must drop them (they are captured again on next use).
static void invalidate_graphs(Server *s) {
  bool any = false;
  for (auto &p : s->pipes) any = any || p.graph_exec;
  if (!any) return;
  (void)hipDeviceSynchronize();
  for (auto &p : s->pipes) {
    if (p.graph_exec) (void)hipGraphExecDestroy(p.graph_exec);
    if (p.graph) (void)hipGraphDestroy(p.graph);
    p.graph_exec = nullptr;
    p.graph = nullptr;
    p.begin_node = nullptr;
  }
}

static int check_pipe(Server *s, int pipe) {
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  if (pipe < 0 || pipe >= (int)s->pipes.size()) LMI_FAIL(LMI_ERR_ARG, "pipe %d out of range", pipe);
  return LMI_OK;
}

template <typename T>
static int dmalloc(T **p, int64_t count) {
  LMI_HIP(hipMalloc((void **)p, (size_t)std::max<int64_t>(count, 1) * sizeof(T)));
  return LMI_OK;
}

static void pipe_free(Pipe &p) {
  void *ptrs[] = {p.ids, p.features, p.labels, p.agg_src_ids, p.agg_src_off, p.agg_dst_off, p.blk_indptr[0],
                  p.blk_indptr[1], p.blk_indptr[2], p.cache_index, p.st, p.dedup.slots, p.eslot[0], p.eslot[1],
                  p.miss_list, p.lru_fill, p.lru_next, p.seed_stage,
                  p.chain_status[0], p.chain_status[1]};
  for (void *q : ptrs)
    if (q) (void)hipFree(q);
  if (p.graph_exec) (void)hipGraphExecDestroy(p.graph_exec);
  if (p.graph) (void)hipGraphDestroy(p.graph);
  if (p.fork) (void)hipEventDestroy(p.fork);
  if (p.fork_early) (void)hipEventDestroy(p.fork_early);
  if (p.join) (void)hipEventDestroy(p.join);
  if (p.handover) (void)hipEventDestroy(p.handover);
  p = Pipe{};
}

// Size of a batch's dedup table: load factor <= 2/3 in the worst case (every sampled edge a new
// node); real batches fill a few percent, and a smaller table is cheaper to clear and to probe.
static int dedup_log2cap(const Server *s) {
  int lg = 4;
  while ((int64_t(1) << lg) * 2 < 3 * s->max_nodes) ++lg;
  return lg;
}

// Status words a look-back scan chain needs: the finest tiling any scan kernel uses, 256 items
// per tile over nodes or edges, or the node tiles of the fused count-and-sample kernel.
static int32_t scan_max_tiles(const Server *s) {
  const int64_t scan_n = std::max(s->max_nodes, s->max_edges_hop);
  int64_t tiles = ceil_div(scan_n, 256);
  for (int k = 0; k < s->cfg.hops; ++k) {
    int G = 4;
    while (G < s->cfg.fanout[k]) G <<= 1;
    tiles = std::max(tiles, ceil_div(s->node_cap[k], (int64_t)std::min(64, 256 / G)));  // smallest tile
  }
  return (int32_t)tiles + 1;
}

static int pipe_alloc(Server *s, Pipe &p) {
  LMI_TRY(dmalloc(&p.ids, s->max_nodes));
  LMI_HIP(hipMalloc(&p.features, (size_t)s->max_nodes * s->row_bytes));
  LMI_TRY(dmalloc(&p.labels, s->cfg.batch_size));
  LMI_TRY(dmalloc(&p.agg_src_ids, s->max_edges));
  LMI_TRY(dmalloc(&p.agg_src_off, s->max_edges));
  LMI_TRY(dmalloc(&p.agg_dst_off, s->max_edges));
  for (int k = 0; k < s->cfg.hops; ++k) LMI_TRY(dmalloc(&p.blk_indptr[k], s->node_cap[k] + 1));
  LMI_TRY(dmalloc(&p.cache_index, s->max_nodes));
  LMI_TRY(dmalloc(&p.st, 1));
  LMI_HIP(hipMemset(p.st, 0, sizeof(DevState)));
  const int lg = dedup_log2cap(s);
  p.dedup.log2cap = lg;
  LMI_HIP(hipMalloc(&p.dedup.slots, size_t(8) << lg));
  LMI_TRY(dmalloc(&p.eslot[0], s->max_edges_hop));
  LMI_TRY(dmalloc(&p.eslot[1], s->max_edges_hop));
  p.max_tiles = scan_max_tiles(s);
  LMI_TRY(dmalloc(&p.chain_status[0], p.max_tiles));
  LMI_TRY(dmalloc(&p.chain_status[1], p.max_tiles));
  LMI_TRY(dmalloc(&p.miss_list, s->max_nodes));
  LMI_TRY(dmalloc(&p.lru_fill, s->max_nodes));
  LMI_TRY(dmalloc(&p.lru_next, s->max_nodes));
  LMI_TRY(dmalloc(&p.seed_stage, s->cfg.batch_size));
  LMI_HIP(hipEventCreateWithFlags(&p.fork, hipEventDisableTiming));
  LMI_HIP(hipEventCreateWithFlags(&p.fork_early, hipEventDisableTiming));
  LMI_HIP(hipEventCreateWithFlags(&p.join, hipEventDisableTiming));
  LMI_HIP(hipEventCreateWithFlags(&p.handover, hipEventDisableTiming));
  return LMI_OK;
}

// Streaming copy, four 16-byte vectors in flight per lane, each block on one contiguous
// 16 KB chunk at a time, non-temporal both ways: the measured HBM copy ceiling (the best of
// the layouts tried: grid-wide strides between a lane's four vectors lose a quarter).
typedef uint32_t cp_u32x4 __attribute__((ext_vector_type(4)));
template <bool HOSTLINK>  // only names the instantiation that reads pinned host memory, so that profiles tell the two apart
static __global__ __launch_bounds__(256) void copy_kernel(const cp_u32x4 *__restrict__ src, cp_u32x4 *__restrict__ dst,
                                                          size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x * 4;
  for (size_t i = (size_t)blockIdx.x * blockDim.x * 4 + threadIdx.x; i < n; i += stride) {
    cp_u32x4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + (size_t)u * blockDim.x < n) v[u] = __builtin_nontemporal_load(src + i + (size_t)u * blockDim.x);
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (i + (size_t)u * blockDim.x < n) __builtin_nontemporal_store(v[u], dst + i + (size_t)u * blockDim.x);
  }
}

// The copy with a gather's read : write shape but none of its indirection: a lane reads RB bytes and
// writes WB bytes per step (8 : 16 is the int8 -> fp16 gather, 4 : 16 int8 -> fp32, 16 : 16 a row
// mover), four steps in flight, each block on contiguous chunks.  A4 offsets both sides by 4 bytes and
// lets the 16-byte accesses assume no more than 4-byte alignment, as rows of 4 k + 4 bytes force.
typedef uint32_t cp_u32x2 __attribute__((ext_vector_type(2)));
typedef cp_u32x4 cp_u32x4_a4 __attribute__((aligned(4)));
template <int RB> struct StreamIn;
template <> struct StreamIn<16> { typedef cp_u32x4 type; };
template <> struct StreamIn<8> { typedef cp_u32x2 type; };
template <> struct StreamIn<4> { typedef uint32_t type; };
template <int RB, int WB, bool A4>
static __global__ __launch_bounds__(256) void stream_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                            size_t n) {
  typedef typename StreamIn<RB>::type IN;
  typedef typename std::conditional<A4, cp_u32x4_a4, cp_u32x4>::type OUT;
  static_assert(WB % 16 == 0 && (!A4 || RB == 16), "whole 16-byte stores; the unaligned variant is the 16 : 16 one");
  const size_t stride = (size_t)gridDim.x * blockDim.x * 4;
  for (size_t i = (size_t)blockIdx.x * blockDim.x * 4 + threadIdx.x; i < n; i += stride) {
    union {
      IN v;
      OUT o;
      uint32_t w[4];
    } r[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = i + (size_t)u * blockDim.x;
      if (j < n) {
        if (A4) r[u].o = __builtin_nontemporal_load(reinterpret_cast<const OUT *>(src + j * RB));
        else r[u].v = __builtin_nontemporal_load(reinterpret_cast<const IN *>(src + j * RB));
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const size_t j = i + (size_t)u * blockDim.x;
      if (j < n) {
        cp_u32x4 o;
        o.x = r[u].w[0];
        o.y = RB >= 8 ? r[u].w[1] : r[u].w[0] + 1u;
        o.z = RB >= 16 ? r[u].w[2] : r[u].w[0] + 2u;
        o.w = RB >= 16 ? r[u].w[3] : r[u].w[0] + 3u;
#pragma unroll
        for (int k = 0; k < WB / 16; ++k) {
          o.x += (uint32_t)k;
          __builtin_nontemporal_store((OUT)o, reinterpret_cast<OUT *>(dst + j * WB + 16 * k));
        }
      }
    }
  }
}

// The same without the one thing stream_kernel leaves out that no gather can avoid: the rows come from
// places all over a large table.  Row r of the output (contiguous, dst_pitch bytes apart) is row
// hash(r) of a table of 2^log2_src_rows rows src_pitch bytes apart, `upr` units of RB bytes each; the
// source row is computed, not loaded, so nothing waits for an index.  A block takes rows_per_block
// consecutive output rows at a time and its 256 threads walk their units in flat order, four in
// flight per lane -- the access pattern of the tiled gathers, minus table lookups, LDS and barriers.
template <int RB, int WB, bool A4, bool EVERY>
static __global__ __launch_bounds__(256) void row_stream_kernel(const uint8_t *__restrict__ src, uint8_t *__restrict__ dst,
                                                                int64_t n_rows, int upr, int64_t src_pitch,
                                                                int64_t dst_pitch, int log2_src_rows, int rows_per_block) {
  typedef typename StreamIn<RB>::type IN;
  typedef typename std::conditional<A4, cp_u32x4_a4, cp_u32x4>::type OUT;
  const int dq = 256 / upr, dr = 256 % upr;
  const int64_t n_tiles = (n_rows + rows_per_block - 1) / rows_per_block;
  for (int64_t tile = blockIdx.x; tile < n_tiles; tile += gridDim.x) {
    const int64_t row0 = tile * rows_per_block;
    const int nr = (int)(n_rows - row0 < rows_per_block ? n_rows - row0 : rows_per_block);
    const int lim = nr * upr;
    int rr = (int)threadIdx.x / upr, uu = (int)threadIdx.x % upr;
    for (int f0 = threadIdx.x; f0 < lim; f0 += 256 * 4) {
      union {
        IN v;
        OUT o;
        uint32_t w[4];
      } r[4];
      int64_t da[4];
      bool on[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        on[u] = f0 + u * 256 < lim;
        const uint32_t out_row = (uint32_t)(row0 + rr);
        uint32_t h = out_row;  // a 32-bit mixer: places as irregular as the ids of a sampled batch, not evenly spread
        h ^= h >> 16; h *= 0x7feb352du; h ^= h >> 15; h *= 0x846ca68bu; h ^= h >> 16;
        const uint32_t src_row = h >> (32 - log2_src_rows);
        const int64_t sa = (int64_t)src_row * src_pitch + (int64_t)uu * RB;
        da[u] = (int64_t)out_row * dst_pitch + (int64_t)uu * WB;
        if (EVERY || on[u]) {  // EVERY: lanes without a unit load all the same (a row that exists), and only skip the store
          if (A4) r[u].o = __builtin_nontemporal_load(reinterpret_cast<const OUT *>(src + sa));
          else r[u].v = __builtin_nontemporal_load(reinterpret_cast<const IN *>(src + sa));
        }
        uu += dr;
        rr += dq;
        if (uu >= upr) {
          uu -= upr;
          ++rr;
        }
      }
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (on[u]) {
          cp_u32x4 o;
          o.x = r[u].w[0];
          o.y = RB >= 8 ? r[u].w[1] : r[u].w[0] + 1u;
          o.z = RB >= 16 ? r[u].w[2] : r[u].w[0] + 2u;
          o.w = RB >= 16 ? r[u].w[3] : r[u].w[0] + 3u;
#pragma unroll
          for (int k = 0; k < WB / 16; ++k) {
            o.x += (uint32_t)k;
            __builtin_nontemporal_store((OUT)o, reinterpret_cast<OUT *>(dst + da[u] + 16 * k));
          }
        }
    }
  }
}

// ------------------------------------------- scratch of lmi_run_once_static
// One array per GPU: every device that loads this code object holds its own copy at its own
// address, from load until the process ends.  It stands in for the scratch a Pipe allocates at
// server creation, carved at fixed offsets and sized for the limits in the header.  In host code
// the array's NAME is only a handle for hipGetSymbolAddress; what kernels, fills and copies get
// is the device address that call returned for the device in use (StaticScratch::ptr).
constexpr int64_t kStaticLog2Cap = 19;  // 2^19 slots hold 1.5 x LMI_STATIC_MAX_NODES keys
constexpr int64_t kStaticMaxTiles = LMI_STATIC_MAX_NODES / 4 + 32;  // smallest tile: 4 nodes (fan-out 64)
constexpr size_t kOffState = 0;
constexpr size_t kOffTable = 256;
constexpr size_t kOffEslot0 = kOffTable + (size_t(8) << kStaticLog2Cap);
constexpr size_t kOffEslot1 = kOffEslot0 + size_t(4) * LMI_STATIC_MAX_HOP_EDGES;
constexpr size_t kOffChain0 = kOffEslot1 + size_t(4) * LMI_STATIC_MAX_HOP_EDGES;
constexpr size_t kOffChain1 = kOffChain0 + size_t(8) * kStaticMaxTiles;
constexpr size_t kOffMiss = kOffChain1 + size_t(8) * kStaticMaxTiles;
constexpr size_t kStaticUsed = kOffMiss + size_t(8) * LMI_STATIC_MAX_NODES;
static_assert(sizeof(DevState) <= 256, "the batch state has a 256-byte slot at the head of the scratch");
static_assert(kStaticUsed <= LMI_STATIC_SCRATCH_BYTES, "the scratch array is too small for its pieces");
static_assert(kOffEslot0 % 256 == 0 && kOffChain0 % 256 == 0 && kOffChain1 % 256 == 0 && kOffMiss % 256 == 0,
              "every piece starts on a 256-byte boundary");

static __device__ __align__(256) unsigned char scratch[LMI_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 16;
struct StaticScratch {
  unsigned char *ptr = nullptr;  // device address of `scratch` on this device
};
static StaticScratch g_static[kMaxDevices];
static std::mutex g_static_mu;

// Once per device, with that device current (lmi_server_create).
static int static_scratch_setup(int device) {
  if (device < 0 || device >= kMaxDevices) return LMI_OK;  // such a device simply has no static entry point
  std::lock_guard<std::mutex> lock(g_static_mu);
  StaticScratch &sc = g_static[device];
  if (sc.ptr) return LMI_OK;
  unsigned char *ptr = nullptr;
  LMI_HIP(hipGetSymbolAddress((void **)&ptr, HIP_SYMBOL(scratch)));
  if (!ptr) LMI_FAIL(LMI_ERR_HIP, "hipGetSymbolAddress gave no address for the static scratch");
  sc.ptr = ptr;
  return LMI_OK;
}

// The two 16-int headers live in the batch state; the caller of the static entry point owns
// separate arrays for them.
static __global__ void copy_headers_kernel(const DevState *st, int32_t *node_counter, int32_t *edge_counter) {
  const int t = threadIdx.x;
  if (t < 16) node_counter[t] = st->node_counter[t];
  else if (t < 32) edge_counter[t - 16] = st->edge_counter[t - 16];
}

}  // namespace lmi

using namespace lmi;

extern "C" {

int lmi_abi_version(void) { return LMI_ABI_VERSION; }
const char *lmi_last_error(void) { return g_err; }

int lmi_server_create(const lmi_config *cfg, lmi_server **out) {
  if (!cfg || !out) LMI_FAIL(LMI_ERR_ARG, "null argument");
  if (cfg->hops < 1 || cfg->hops > LMI_MAX_HOPS) LMI_FAIL(LMI_ERR_ARG, "hops must be 1..%d", LMI_MAX_HOPS);
  if (cfg->batch_size < 1) LMI_FAIL(LMI_ERR_ARG, "batch_size must be positive");
  if (cfg->feat_dim < 1) LMI_FAIL(LMI_ERR_ARG, "feat_dim must be positive");
  if (cfg->feat_dtype != LMI_F32 && cfg->feat_dtype != LMI_F16) LMI_FAIL(LMI_ERR_ARG, "bad feat_dtype");
  if (cfg->pipes < 1 || cfg->pipes > LMI_MAX_PIPES) LMI_FAIL(LMI_ERR_ARG, "pipes must be 1..%d", LMI_MAX_PIPES);
  for (int k = 0; k < cfg->hops; ++k)
    if (cfg->fanout[k] < 1 || cfg->fanout[k] > LMI_MAX_FANOUT)
      LMI_FAIL(LMI_ERR_ARG, "fanout[%d]=%d outside 1..%d", k, cfg->fanout[k], LMI_MAX_FANOUT);
  int n_dev = 0;
  LMI_HIP(hipGetDeviceCount(&n_dev));
  if (cfg->device_id < 0 || cfg->device_id >= n_dev) LMI_FAIL(LMI_ERR_ARG, "device %d not present", cfg->device_id);
  LMI_HIP(hipSetDevice(cfg->device_id));
  LMI_TRY(static_scratch_setup(cfg->device_id));
  Server *s = new (std::nothrow) Server;
  if (!s) LMI_FAIL(LMI_ERR_HIP, "out of host memory");
  s->cfg = *cfg;
  s->row_bytes = (int64_t)cfg->feat_dim * (cfg->feat_dtype == LMI_F16 ? 2 : 4);
  if (s->row_bytes % 4 != 0) {
    delete s;
    LMI_FAIL(LMI_ERR_ARG, "feature rows must be a multiple of 4 bytes");
  }
  // worst case: n_k <= n_{k-1} * (1 + f_k)   (the reference under-sizes this, engine/server.cu:204-216)
  s->node_cap[0] = cfg->batch_size;
  for (int k = 0; k < cfg->hops; ++k) {
    s->edge_cap[k] = s->node_cap[k] * cfg->fanout[k];
    s->node_cap[k + 1] = s->node_cap[k] + s->edge_cap[k];
    s->max_edges += s->edge_cap[k];
    s->max_edges_hop = std::max(s->max_edges_hop, s->edge_cap[k]);
  }
  for (int k = cfg->hops + 1; k <= LMI_MAX_HOPS; ++k) s->node_cap[k] = s->node_cap[cfg->hops];
  s->max_nodes = s->node_cap[cfg->hops];
  if (s->max_nodes + s->max_edges_hop >= (int64_t(1) << 30)) {
    delete s;
    LMI_FAIL(LMI_ERR_CAPACITY, "batch_size x fanouts too large for 32-bit local ids");
  }
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, cfg->device_id) == hipSuccess) s->n_cu = prop.multiProcessorCount;
  s->pipes.resize(cfg->pipes);
  int rc = LMI_OK;
  for (auto &p : s->pipes)
    if ((rc = pipe_alloc(s, p)) != LMI_OK) break;
  if (rc == LMI_OK && hipMalloc(&s->d_scalar, 64) != hipSuccess) rc = LMI_ERR_HIP;
  if (rc == LMI_OK && hipStreamCreateWithFlags(&s->side, hipStreamNonBlocking) != hipSuccess) rc = LMI_ERR_HIP;
  if (rc == LMI_OK && hipEventCreateWithFlags(&s->lru_ready, hipEventDisableTiming) != hipSuccess) rc = LMI_ERR_HIP;
  if (rc == LMI_OK && hipEventCreateWithFlags(&s->lru_copied, hipEventDisableTiming) != hipSuccess) rc = LMI_ERR_HIP;
  if (rc == LMI_OK && hipEventCreateWithFlags(&s->side_idle, hipEventDisableTiming) != hipSuccess) rc = LMI_ERR_HIP;
  if (rc == LMI_OK && (hipMalloc(&s->d_prof_rows, 16) != hipSuccess || hipMemset(s->d_prof_rows, 0, 16) != hipSuccess))
    rc = LMI_ERR_HIP;
  if (rc == LMI_OK) {  // sticky fault words: pinned host memory the kernels write and the host reads without a copy
    void *fh = nullptr, *fd = nullptr;
    if (hipHostMalloc(&fh, 64, hipHostMallocMapped) != hipSuccess) rc = LMI_ERR_HIP;
    if (rc == LMI_OK) {
      memset(fh, 0, 64);
      s->fault_host = (volatile int32_t *)fh;
      if (hipHostGetDevicePointer(&fd, fh, 0) != hipSuccess) rc = LMI_ERR_HIP;
      s->fault_dev = (int32_t *)fd;
      s->rows_seen_host = s->fault_host + 8;  // the second half of the 64 bytes
      s->rows_seen_dev = s->fault_dev ? s->fault_dev + 8 : nullptr;
    }
  }
  if (rc != LMI_OK) {
    lmi_server_destroy(reinterpret_cast<lmi_server *>(s));
    return rc;
  }
  *out = reinterpret_cast<lmi_server *>(s);
  return LMI_OK;
}

int lmi_server_pipes(lmi_server *h, int32_t pipes) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  if (pipes < 1 || pipes > LMI_MAX_PIPES) LMI_FAIL(LMI_ERR_ARG, "pipes must be 1..%d", LMI_MAX_PIPES);
  const size_t have = s->pipes.size();
  if ((size_t)pipes <= have) return LMI_OK;  // never shrinks: callers may hold views of the existing sets
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  s->pipes.resize((size_t)pipes);  // moves the host-side records only; device buffers stay where they are
  int rc = LMI_OK;
  for (size_t k = have; k < s->pipes.size() && rc == LMI_OK; ++k) rc = pipe_alloc(s, s->pipes[k]);
  if (rc != LMI_OK) {
    for (size_t k = have; k < s->pipes.size(); ++k) pipe_free(s->pipes[k]);
    s->pipes.resize(have);
    return rc;
  }
  s->cfg.pipes = pipes;
  return LMI_OK;
}

int lmi_server_destroy(lmi_server *h) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) return LMI_OK;
  (void)hipSetDevice(s->cfg.device_id);
  (void)hipDeviceSynchronize();
  for (auto &p : s->pipes) pipe_free(p);
  cache_free(s);
  if (s->own_graph) {
    (void)hipFree((void *)s->indptr);
    (void)hipFree((void *)s->indices);
  }
  for (int m = 0; m < 3; ++m) {
    if (s->set_ids[m]) (void)hipFree(s->set_ids[m]);
    if (s->set_labels[m]) (void)hipFree(s->set_labels[m]);
  }
  for (auto &e : s->prof_used) (void)hipEventDestroy(e);
  for (auto &e : s->prof_free) (void)hipEventDestroy(e);
  if (s->d_prof_rows) (void)hipFree(s->d_prof_rows);
  if (s->d_scalar) (void)hipFree(s->d_scalar);
  if (s->hot) (void)hipFree(s->hot);
  if (s->side) (void)hipStreamDestroy(s->side);
  if (s->lru_ready) (void)hipEventDestroy(s->lru_ready);
  if (s->lru_copied) (void)hipEventDestroy(s->lru_copied);
  if (s->side_idle) (void)hipEventDestroy(s->side_idle);
  if (s->fault_host) (void)hipHostFree((void *)s->fault_host);
  delete s;
  return LMI_OK;
}

// ------------------------------------------------------------ memory helpers
int lmi_host_alloc(size_t bytes, void **host_ptr) {
  if (!host_ptr) LMI_FAIL(LMI_ERR_ARG, "null argument");
  LMI_HIP(hipHostMalloc(host_ptr, bytes ? bytes : 1, hipHostMallocMapped | hipHostMallocPortable));
  return LMI_OK;
}
int lmi_host_free(void *host_ptr) {
  if (host_ptr) LMI_HIP(hipHostFree(host_ptr));
  return LMI_OK;
}
int lmi_device_alloc(size_t bytes, void **dev_ptr) {
  if (!dev_ptr) LMI_FAIL(LMI_ERR_ARG, "null argument");
  LMI_HIP(hipMalloc(dev_ptr, bytes ? bytes : 1));
  return LMI_OK;
}
int lmi_device_free(void *dev_ptr) {
  if (dev_ptr) LMI_HIP(hipFree(dev_ptr));
  return LMI_OK;
}
int lmi_copy_to_host(void *host_dst, const void *dev_src, size_t bytes) {
  LMI_HIP(hipMemcpy(host_dst, dev_src, bytes, hipMemcpyDeviceToHost));
  return LMI_OK;
}
int lmi_copy_to_device(void *dev_dst, const void *host_src, size_t bytes) {
  LMI_HIP(hipMemcpy(dev_dst, host_src, bytes, hipMemcpyHostToDevice));
  return LMI_OK;
}
int lmi_copy_device(void *dev_dst, const void *dev_src, size_t bytes, void *stream) {
  if (bytes) LMI_HIP(hipMemcpyAsync(dev_dst, dev_src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream));
  return LMI_OK;
}
int lmi_ipc_export(const void *dev_ptr, void *handle, int64_t *offset, int64_t *alloc_bytes) {
  static_assert(sizeof(hipIpcMemHandle_t) == LMI_IPC_HANDLE_BYTES, "the handle slot is sized for hipIpcMemHandle_t");
  if (!dev_ptr || !handle) LMI_FAIL(LMI_ERR_ARG, "null argument");
  hipDeviceptr_t base = nullptr;
  size_t size = 0;
  LMI_HIP(hipMemGetAddressRange(&base, &size, (hipDeviceptr_t)const_cast<void *>(dev_ptr)));
  if ((int64_t)size >= LMI_IPC_MAX_BYTES)
    LMI_FAIL(LMI_ERR_CAPACITY, "an allocation of %zu bytes cannot be shared with another process (limit %lld): split it",
             size, (long long)LMI_IPC_MAX_BYTES);
  hipIpcMemHandle_t h;
  LMI_HIP(hipIpcGetMemHandle(&h, (void *)base));
  memcpy(handle, &h, sizeof(h));
  if (offset) *offset = (int64_t)((const char *)dev_ptr - (const char *)base);
  if (alloc_bytes) *alloc_bytes = (int64_t)size;
  return LMI_OK;
}
int lmi_ipc_open(const void *handle, void **dev_base) {
  if (!handle || !dev_base) LMI_FAIL(LMI_ERR_ARG, "null argument");
  hipIpcMemHandle_t h;
  memcpy(&h, handle, sizeof(h));
  LMI_HIP(hipIpcOpenMemHandle(dev_base, h, hipIpcMemLazyEnablePeerAccess));
  return LMI_OK;
}
int lmi_ipc_close(void *dev_base) {
  if (dev_base) LMI_HIP(hipIpcCloseMemHandle(dev_base));
  return LMI_OK;
}
int lmi_stream_create(void **stream) {
  if (!stream) LMI_FAIL(LMI_ERR_ARG, "null argument");
  hipStream_t st;
  LMI_HIP(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
  *stream = st;
  return LMI_OK;
}
int lmi_stream_destroy(void *stream) {
  if (stream) LMI_HIP(hipStreamDestroy((hipStream_t)stream));
  return LMI_OK;
}
int lmi_stream_sync(void *stream) {
  LMI_HIP(hipStreamSynchronize((hipStream_t)stream));
  return LMI_OK;
}
int lmi_device_sync(void) {
  LMI_HIP(hipDeviceSynchronize());
  return LMI_OK;
}

// ------------------------------------------------------------------ storage
int lmi_graph_load(lmi_server *h, const int64_t *indptr, const int32_t *indices, int64_t n_nodes, int64_t n_edges,
                   int location) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !indptr || (!indices && n_edges > 0)) LMI_FAIL(LMI_ERR_ARG, "null argument");
  if (n_nodes < 1 || n_nodes >= (int64_t(1) << 31) - 4096 || n_edges < 0) LMI_FAIL(LMI_ERR_ARG, "bad graph size");
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  invalidate_graphs(s);
  if (s->own_graph) {
    (void)hipFree((void *)s->indptr);
    (void)hipFree((void *)s->indices);
    s->own_graph = false;
  }
  if (s->hot) {  // counts belong to the previous graph
    (void)hipFree(s->hot);
    s->hot = nullptr;
  }
  if (location == LMI_LOC_DEVICE) {
    s->indptr = indptr;
    s->indices = indices;
  } else if (location == LMI_LOC_HOST) {
    if (indptr[0] != 0 || indptr[n_nodes] != n_edges) LMI_FAIL(LMI_ERR_ARG, "indptr[0] must be 0 and indptr[n] == n_edges");
    int64_t *dp = nullptr;
    int32_t *di = nullptr;
    LMI_HIP(hipMalloc(&dp, (size_t)(n_nodes + 1) * 8));
    LMI_HIP(hipMalloc(&di, (size_t)std::max<int64_t>(n_edges, 1) * 4));
    LMI_HIP(hipMemcpy(dp, indptr, (size_t)(n_nodes + 1) * 8, hipMemcpyHostToDevice));
    if (n_edges) LMI_HIP(hipMemcpy(di, indices, (size_t)n_edges * 4, hipMemcpyHostToDevice));
    s->indptr = dp;
    s->indices = di;
    s->own_graph = true;
  } else {
    LMI_FAIL(LMI_ERR_ARG, "bad location");
  }
  s->n_nodes = n_nodes;
  s->n_edges = n_edges;
  return LMI_OK;
}

int lmi_features_attach(lmi_server *h, const void *rows, int64_t n_rows, int location) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !rows || n_rows < 1) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  if (location == LMI_LOC_HOST) {
    void *d = nullptr;
    if (hipHostGetDevicePointer(&d, const_cast<void *>(rows), 0) != hipSuccess) {
      (void)hipGetLastError();
      LMI_FAIL(LMI_ERR_ARG, "host feature rows must be allocated with lmi_host_alloc (pinned + mapped)");
    }
    s->feat = (const uint8_t *)d;
  } else if (location == LMI_LOC_DEVICE) {
    s->feat = (const uint8_t *)rows;
  } else {
    LMI_FAIL(LMI_ERR_ARG, "bad location");
  }
  s->feat_rows = n_rows;
  s->feat_loc = location;
  return LMI_OK;
}

int lmi_idset_load(lmi_server *h, int mode, const int32_t *ids, const int32_t *labels, int64_t n, int location) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !ids || n < 1 || mode < 0 || mode > 2) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  const hipMemcpyKind kind = location == LMI_LOC_DEVICE ? hipMemcpyDeviceToDevice : hipMemcpyHostToDevice;
  if (s->set_ids[mode]) (void)hipFree(s->set_ids[mode]);
  if (s->set_labels[mode]) (void)hipFree(s->set_labels[mode]);
  s->set_ids[mode] = s->set_labels[mode] = nullptr;
  LMI_HIP(hipMalloc(&s->set_ids[mode], (size_t)n * 4));
  LMI_HIP(hipMemcpy(s->set_ids[mode], ids, (size_t)n * 4, kind));
  if (labels) {
    LMI_HIP(hipMalloc(&s->set_labels[mode], (size_t)n * 4));
    LMI_HIP(hipMemcpy(s->set_labels[mode], labels, (size_t)n * 4, kind));
  }
  s->set_n[mode] = n;
  return LMI_OK;
}

// ------------------------------------------------------------------- caches
int lmi_cache_build_static(lmi_server *h, int64_t capacity_rows, int table_kind) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  invalidate_graphs(s);
  return cache_build_static(s, capacity_rows, table_kind, false);
}
int lmi_cache_build_int8(lmi_server *h, int64_t capacity_rows, int table_kind) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  invalidate_graphs(s);
  return cache_build_static(s, capacity_rows, table_kind, true);
}
int lmi_cache_build_lru(lmi_server *h, int64_t n_sets, int32_t ways) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  invalidate_graphs(s);
  return cache_build_lru(s, n_sets, ways);
}
int lmi_cache_info_get(lmi_server *h, lmi_cache_info *out) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !out) LMI_FAIL(LMI_ERR_ARG, "null argument");
  memset(out, 0, sizeof(*out));
  out->kind = s->cache_kind;
  out->table_kind = s->table_kind;
  out->capacity_rows = s->cache_rows;
  out->row_bytes = s->cache_row_bytes;
  out->table_bytes = s->cache_kind == LMI_CACHE_LRU ? s->cache_rows * 8
                     : s->table_kind == LMI_TABLE_DIRECT ? (s->slot_of ? s->n_nodes * 4 : 0)
                     : s->table_kind == LMI_TABLE_RANK ? (s->rank_tab ? ceil_div(s->n_nodes, 64) * 16 : 0)
                                                         : (int64_t)s->id_table.bytes();
  out->n_sets = s->lru_sets;
  out->ways = s->lru_ways;
  out->lru_tick = s->lru_tick;
  return LMI_OK;
}
int lmi_cache_dump(lmi_server *h, int32_t *slot_of, int64_t n, int32_t *aux) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !slot_of) LMI_FAIL(LMI_ERR_ARG, "null argument");
  LMI_HIP(hipSetDevice(s->cfg.device_id));
  return cache_dump(s, slot_of, n, aux);
}

// -------------------------------------------------------------- presampling
int lmi_cache_policy(lmi_server *h, int policy) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || (policy != LMI_POLICY_DEGREE && policy != LMI_POLICY_PRESAMPLED)) LMI_FAIL(LMI_ERR_ARG, "bad policy");
  s->policy = policy;
  return LMI_OK;
}

int lmi_presample_reset(lmi_server *h) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  LMI_HIP(hipDeviceSynchronize());
  if (s->hot) LMI_HIP(hipMemset(s->hot, 0, (size_t)s->n_nodes * 4));
  return LMI_OK;
}

int lmi_hotness_dump(lmi_server *h, uint32_t *counts, int64_t n) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !counts || n != s->n_nodes) LMI_FAIL(LMI_ERR_ARG, "hotness dump needs n == n_nodes");
  if (!s->hot) LMI_FAIL(LMI_ERR_STATE, "nothing presampled yet");
  LMI_HIP(hipDeviceSynchronize());
  LMI_HIP(hipMemcpy(counts, s->hot, (size_t)n * 4, hipMemcpyDeviceToHost));
  return LMI_OK;
}

// ---------------------------------------------------------------- operators
static int ready(Server *s) {
  if (!s->indptr) LMI_FAIL(LMI_ERR_STATE, "no graph loaded");
  return LMI_OK;
}

// Resolves where this batch's seeds live and the per-batch scalars.
static int batch_params(Server *s, Pipe &p, hipStream_t st, const int32_t *seeds, int32_t n, int seeds_location,
                        int32_t batch_counter, int mode, uint64_t rng_seed, BatchParams *bp) {
  LMI_TRY(ready(s));
  bp->labels = nullptr;
  if (seeds) {
    if (n < 0 || n > s->cfg.batch_size) LMI_FAIL(LMI_ERR_CAPACITY, "%d seeds exceed batch_size %d", n, s->cfg.batch_size);
    if (seeds_location == LMI_LOC_DEVICE) bp->seeds = seeds;
    else {
      if (n) LMI_HIP(hipMemcpyAsync(p.seed_stage, seeds, (size_t)n * 4, hipMemcpyHostToDevice, st));
      bp->seeds = p.seed_stage;
    }
  } else {
    // slice `batch_counter` of the id set (batch_generate, operator_impl.cu:40-53); a short last
    // batch is shortened rather than padded with -1
    if (mode < 0 || mode > 2 || !s->set_ids[mode]) LMI_FAIL(LMI_ERR_STATE, "id set %d not loaded", mode);
    const int32_t per = s->set_batch[mode] ? s->set_batch[mode] : s->cfg.batch_size;
    const int64_t off = (int64_t)batch_counter * per;
    if (batch_counter < 0 || off >= s->set_n[mode]) LMI_FAIL(LMI_ERR_ARG, "batch %d is past the end of id set %d", batch_counter, mode);
    n = (int32_t)std::min<int64_t>(per, s->set_n[mode] - off);
    bp->seeds = s->set_ids[mode] + off;
    if (s->set_labels[mode]) bp->labels = s->set_labels[mode] + off;
  }
  bp->n_seeds = n;
  // dedup-table epoch: keys carry it in the bits above the widest node id, so the table is
  // wiped only when the epochs run out (or it is new, or the id width changed)
  int id_bits = 1;
  while (id_bits < 31 && (int64_t(1) << id_bits) < s->n_nodes) ++id_bits;
  const int32_t max_epoch = (int32_t)std::min<int64_t>((int64_t(1) << (31 - id_bits)) - 1, s->table_epochs);  // 0: wipe every batch
  if (p.table_dirty || p.epoch >= max_epoch || p.id_bits != id_bits) {
    p.epoch = 0;
    bp->clear_table = 1;
  } else {
    ++p.epoch;
    bp->clear_table = 0;
  }
  p.table_dirty = false;
  p.id_bits = id_bits;
  bp->table_tag = max_epoch > 0 ? (int32_t)((uint32_t)p.epoch << id_bits) : 0;
  bp->table_mask = max_epoch > 0 ? (int32_t)(0xFFFFFFFFu << id_bits) : kUntaggedMask;
  bp->fault = s->fault_dev;
  bp->rng_seed = rng_seed ? rng_seed : s->cfg.seed + (uint64_t)(uint32_t)batch_counter;
  if (s->cache_kind == LMI_CACHE_LRU) ++s->lru_tick;
  bp->lru_tick = s->lru_tick;
  return LMI_OK;
}

int lmi_op_batch_generate(lmi_server *h, int pipe, void *stream, const int32_t *seeds, int32_t n, int seeds_location,
                          int32_t batch_counter, int mode, uint64_t rng_seed) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  Pipe &p = s->pipes[pipe];
  hipStream_t st = (hipStream_t)stream;
  BatchParams bp{};
  prof_batch(s);
  LMI_TRY(pipe_join(p, st));
  pipe_begin(p, st);
  LMI_TRY(batch_params(s, p, st, seeds, n, seeds_location, batch_counter, mode, rng_seed, &bp));
  Pipe *pp[1] = {&p};
  return launch_batch_generate(s, pp, &bp, 1, st, true);
}

int lmi_op_random_sample(lmi_server *h, int pipe, void *stream, int hop) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  LMI_TRY(ready(s));
  Pipe &p = s->pipes[pipe];
  if (hop != p.hops_done || hop >= s->cfg.hops) LMI_FAIL(LMI_ERR_ARG, "hop %d out of order (next is %d)", hop, p.hops_done);
  hipStream_t st = (hipStream_t)stream;
  LMI_TRY(pipe_handover(p, st));  // a stream other than the one of the operator before is ordered behind it
  pipe_begin(p, st);
  prof_phase(s, st, &s->prof_open, PROF_SAMPLE);
  Pipe *pp[1] = {&p};
  LMI_TRY(launch_hop(s, pp, 1, st, hop, false, false));
  prof_phase(s, st, &s->prof_open, -1);
  return LMI_OK;
}

int lmi_op_cache_lookup(lmi_server *h, int pipe, void *stream, int segment) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  if (!s->feat) LMI_FAIL(LMI_ERR_STATE, "no features attached");
  Pipe &p = s->pipes[pipe];
  if (segment < 0 || segment > p.hops_done) LMI_FAIL(LMI_ERR_ARG, "segment %d not sampled yet", segment);
  hipStream_t st = (hipStream_t)stream;
  LMI_TRY(pipe_join(p, st));
  pipe_begin(p, st);
  LMI_TRY(lru_wait_ready(s, st));
  prof_phase(s, st, &s->prof_open, PROF_LOOKUP);
  Pipe *pp[1] = {&p};
  LMI_TRY(launch_lookup(s, pp, 1, st, segment, segment));
  LMI_TRY(launch_gather_seg(s, p, st, segment, segment, 0));
  prof_phase(s, st, &s->prof_open, -1);
  return LMI_OK;
}

int lmi_op_hotness(lmi_server *h, int pipe, void *stream) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  LMI_TRY(ready(s));
  LMI_TRY(pipe_join(s->pipes[pipe], (hipStream_t)stream));
  pipe_begin(s->pipes[pipe], (hipStream_t)stream);
  return launch_hotness(s, s->pipes[pipe], (hipStream_t)stream);
}

int lmi_presample(lmi_server *h, int pipe, void *stream, int mode, int32_t first_batch, int32_t n_batches) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  if (n_batches < 0) LMI_FAIL(LMI_ERR_ARG, "negative batch count");
  Pipe &p = s->pipes[pipe];
  hipStream_t st = (hipStream_t)stream;
  for (int32_t b = first_batch; b < first_batch + n_batches; ++b) {
    BatchParams bp{};
    LMI_TRY(pipe_join(p, st));
    pipe_begin(p, st);
    const int tick = s->lru_tick;
    LMI_TRY(batch_params(s, p, st, nullptr, 0, LMI_LOC_DEVICE, b, mode, 0, &bp));
    s->lru_tick = tick;  // presampling does not age the LRU cache
    Pipe *pp[1] = {&p};
    LMI_TRY(launch_batch_generate(s, pp, &bp, 1, st, false));
    for (int k = 0; k < s->cfg.hops; ++k) LMI_TRY(launch_hop(s, pp, 1, st, k, true, true));
    LMI_TRY(launch_fill(s, pp, 1, st));
    LMI_TRY(launch_hotness(s, p, st));
  }
  return LMI_OK;
}

int lmi_op_io_submit(lmi_server *h, int pipe, void *stream) {
  (void)stream;
  return check_pipe(reinterpret_cast<Server *>(h), pipe);
}

int lmi_op_io_complete(lmi_server *h, int pipe, void *stream) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  Pipe &p = s->pipes[pipe];
  hipStream_t st = (hipStream_t)stream;
  LMI_TRY(pipe_join(p, st));
  pipe_begin(p, st);
  LMI_TRY(launch_lru_insert(s, p, st, s->cfg.hops + 1));
  return LMI_OK;
}

// Captures begin + hops + lookup of one pipe into a HIP graph.  Every kernel in it
// reads its sizes and per-batch scalars from the pipe's DevState, so a replay only
// needs the first node (batch_begin_kernel) re-pointed at the new batch.
static int capture_batch_graph(Server *s, Pipe &p, hipStream_t st, const BatchParams &bp) {
  const bool prof = s->prof_on;
  s->prof_on = false;  // no event records inside the capture
  LMI_HIP(hipStreamBeginCapture(st, hipStreamCaptureModeThreadLocal));
  Pipe *pp[1] = {&p};
  int rc = launch_batch_generate(s, pp, &bp, 1, st, false);
  for (int k = 0; rc == LMI_OK && k < s->cfg.hops; ++k) rc = launch_hop(s, pp, 1, st, k, true, true);
  if (rc == LMI_OK) rc = launch_lookup(s, pp, 1, st, 0, s->cfg.hops);
  hipGraph_t g = nullptr;
  const hipError_t e = hipStreamEndCapture(st, &g);
  s->prof_on = prof;
  if (rc != LMI_OK) {
    if (g) (void)hipGraphDestroy(g);
    return rc;
  }
  LMI_HIP(e);
  size_t n_roots = 1;
  hipGraphNode_t root = nullptr;
  LMI_HIP(hipGraphGetRootNodes(g, &root, &n_roots));
  hipGraphNodeType ty;
  LMI_HIP(hipGraphNodeGetType(root, &ty));
  if (n_roots != 1 || ty != hipGraphNodeTypeKernel) {
    (void)hipGraphDestroy(g);
    LMI_FAIL(LMI_ERR_HIP, "captured batch graph has an unexpected shape (%zu roots)", n_roots);
  }
  LMI_HIP(hipGraphInstantiate(&p.graph_exec, g, nullptr, nullptr, 0));
  p.graph = g;
  p.begin_node = root;
  return LMI_OK;
}

// One batch on each of n pipes, served by the same launches.
// The caller has ordered `st` behind the pipes' previous batches (pipes_join) before it staged the seeds.
static int run_group(Server *s, Pipe *const *pp, const BatchParams *bps, int n, hipStream_t st) {
  for (int k = 0; k < n; ++k) pipe_begin(*pp[k], st);
  prof_phase(s, st, &s->prof_open, PROF_SAMPLE);
  bool split = false;
  if (s->use_graph && st != nullptr && n == 1) {  // the legacy default stream cannot be captured
    Pipe &p = *pp[0];
    LMI_TRY(lru_wait_ready(s, st));  // the lookup sits inside the graph: the whole replay waits
    if (!p.graph_exec) LMI_TRY(capture_batch_graph(s, p, st, bps[0]));
    LMI_TRY(graph_update_begin(s, p, bps[0]));
    LMI_HIP(hipGraphLaunch(p.graph_exec, st));
  } else {
    // split_lookup: the seeds and the first hop's nodes are looked up as soon as they are known and their
    // misses start over the host link while the later hops are still being sampled
    split = s->split_lookup && s->cfg.hops >= 2 && s->feat_loc == LMI_LOC_HOST && s->split_miss == 1 &&
            (s->cache_kind == LMI_CACHE_STATIC || s->cache_kind == LMI_CACHE_INT8) &&
            (s->split_lookup == 1 || (s->split_lookup == 2 && n > 1));
    LMI_TRY(launch_batch_generate(s, pp, bps, n, st, false));
    for (int k = 0; k < s->cfg.hops; ++k) {
      LMI_TRY(launch_hop(s, pp, n, st, k, true, true));
      if (split && k == 0) {
        LMI_TRY(launch_lookup(s, pp, n, st, 0, 1));
        LMI_TRY(launch_misses_early(s, pp, n, st, 0, 1));
      }
    }
    LMI_TRY(lru_wait_ready(s, st));  // sampling may overlap the previous batch's insertion, the lookup may not
    LMI_TRY(launch_lookup(s, pp, n, st, split ? 2 : 0, s->cfg.hops));
  }
  LMI_TRY(launch_gather_group(s, pp, n, st, split ? 2 : 0, s->cfg.hops, s->cache_kind == LMI_CACHE_LRU ? 1 : 0, false, 0));
  prof_phase(s, st, &s->prof_open, -1);
  return LMI_OK;
}

int lmi_run_once(lmi_server *h, int pipe, void *stream, const int32_t *seeds, int32_t n, int seeds_location,
                 int32_t batch_counter, int mode, uint64_t rng_seed) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  if (!s->feat) LMI_FAIL(LMI_ERR_STATE, "no features attached");
  Pipe *pp[1] = {&s->pipes[pipe]};
  hipStream_t st = (hipStream_t)stream;
  BatchParams bp{};
  prof_batch(s);
  // a pipe's previous batch may still be gathering misses, or sit on another stream: only behind it may
  // this batch's first command, the copy of host seeds into the pipe's staging buffer, be queued
  LMI_TRY(pipes_join(pp, 1, st));
  LMI_TRY(batch_params(s, *pp[0], st, seeds, n, seeds_location, batch_counter, mode, rng_seed, &bp));
  return run_group(s, pp, &bp, 1, st);
}

int lmi_run_group(lmi_server *h, int n_batches, const int32_t *pipes, void *stream, const int32_t *const *seeds,
                  const int32_t *n_seeds, int seeds_location, const int32_t *batch_counters, int mode,
                  const uint64_t *rng_seeds) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !pipes || !batch_counters) LMI_FAIL(LMI_ERR_ARG, "null argument");
  if (n_batches < 1 || n_batches > LMI_MAX_GROUP) LMI_FAIL(LMI_ERR_ARG, "a group holds 1..%d batches", LMI_MAX_GROUP);
  if (!s->feat) LMI_FAIL(LMI_ERR_STATE, "no features attached");
  if (s->cache_kind == LMI_CACHE_LRU && n_batches > 1)
    LMI_FAIL(LMI_ERR_STATE, "the LRU cache takes one batch at a time (its state is batch-synchronous)");
  Pipe *pp[LMI_MAX_GROUP];
  BatchParams bps[LMI_MAX_GROUP];
  hipStream_t st = (hipStream_t)stream;
  for (int k = 0; k < n_batches; ++k) {
    LMI_TRY(check_pipe(s, pipes[k]));
    for (int j = 0; j < k; ++j)
      if (pipes[j] == pipes[k]) LMI_FAIL(LMI_ERR_ARG, "pipe %d named twice in one group", pipes[k]);
    pp[k] = &s->pipes[pipes[k]];
  }
  prof_batch(s, n_batches);
  LMI_TRY(pipes_join(pp, n_batches, st));  // before the seeds are staged: see lmi_run_once
  for (int k = 0; k < n_batches; ++k)
    LMI_TRY(batch_params(s, *pp[k], st, seeds ? seeds[k] : nullptr, (seeds && n_seeds) ? n_seeds[k] : 0, seeds_location,
                         batch_counters[k], mode, rng_seeds ? rng_seeds[k] : 0, &bps[k]));
  return run_group(s, pp, bps, n_batches, st);
}

int lmi_run_once_static(lmi_server *h, void *stream, const int32_t *seeds, int32_t n, uint64_t rng_seed,
                        const lmi_batch_view *out) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !out || !seeds) LMI_FAIL(LMI_ERR_ARG, "null argument");
  if (!s->feat) LMI_FAIL(LMI_ERR_STATE, "no features attached");
  if (s->cache_kind == LMI_CACHE_LRU)
    LMI_FAIL(LMI_ERR_STATE, "the LRU cache keeps per-pipe insertion state: use lmi_run_once");
  if (s->max_nodes > LMI_STATIC_MAX_NODES || s->max_edges_hop > LMI_STATIC_MAX_HOP_EDGES)
    LMI_FAIL(LMI_ERR_CAPACITY,
             "this server's worst case (%lld rows per batch, %lld edges in a hop) exceeds the static scratch "
             "(%d rows, %d edges): use lmi_run_once", (long long)s->max_nodes, (long long)s->max_edges_hop,
             LMI_STATIC_MAX_NODES, LMI_STATIC_MAX_HOP_EDGES);
  const int lg = dedup_log2cap(s);
  const int32_t tiles = scan_max_tiles(s);
  if (lg > kStaticLog2Cap || tiles > kStaticMaxTiles)
    LMI_FAIL(LMI_ERR_CAPACITY, "this server's scan tiles or dedup table exceed the static scratch");
  bool have = out->ids && out->features && out->labels && out->agg_src_ids && out->agg_src_off && out->agg_dst_off &&
              out->node_counter && out->edge_counter && out->cache_index;
  for (int k = 0; k < s->cfg.hops; ++k) have = have && out->blk_indptr[k];
  if (!have) LMI_FAIL(LMI_ERR_ARG, "every output buffer of the view must be given");
  if (out->max_nodes < s->max_nodes || out->max_edges < s->max_edges)
    LMI_FAIL(LMI_ERR_CAPACITY, "the output buffers must hold the worst case: %lld rows, %lld edges",
             (long long)s->max_nodes, (long long)s->max_edges);
  if ((uintptr_t)out->features % 16 != 0) LMI_FAIL(LMI_ERR_ARG, "the feature buffer must be 16-byte aligned");
  const int device = s->cfg.device_id;
  if (device < 0 || device >= kMaxDevices || !g_static[device].ptr)
    LMI_FAIL(LMI_ERR_STATE, "no static scratch on device %d", device);
  LMI_HIP(hipSetDevice(device));
  unsigned char *ptr = g_static[device].ptr;
  // The "pipe" of this call lives on the stack: nothing of it outlasts the call, so two servers on one
  // GPU share the device array (the documented race) but no host-side state.  Its table is wiped by
  // every call (no epoch kept on the host): another server may have used the array last, and the
  // launches of a call must depend on nothing but its arguments and the device memory they name, so
  // that a caller who captured them in a graph can replay it.
  Pipe p;
  p.table_dirty = true;
  p.ids = out->ids;
  p.features = out->features;
  p.labels = out->labels;
  p.agg_src_ids = out->agg_src_ids;
  p.agg_src_off = out->agg_src_off;
  p.agg_dst_off = out->agg_dst_off;
  for (int k = 0; k < LMI_MAX_HOPS; ++k) p.blk_indptr[k] = out->blk_indptr[k];
  p.cache_index = out->cache_index;
  p.st = reinterpret_cast<DevState *>(ptr + kOffState);
  p.dedup.slots = reinterpret_cast<HashSlot *>(ptr + kOffTable);
  p.dedup.log2cap = lg;
  p.eslot[0] = reinterpret_cast<int32_t *>(ptr + kOffEslot0);
  p.eslot[1] = reinterpret_cast<int32_t *>(ptr + kOffEslot1);
  p.chain_status[0] = reinterpret_cast<unsigned long long *>(ptr + kOffChain0);
  p.chain_status[1] = reinterpret_cast<unsigned long long *>(ptr + kOffChain1);
  p.max_tiles = tiles;
  p.miss_list = reinterpret_cast<int2 *>(ptr + kOffMiss);
  p.fill_pending = -1;
  p.side_pending = false;
  hipStream_t st = (hipStream_t)stream;
  Pipe *pp[1] = {&p};
  BatchParams bp{};
  const bool prof = s->prof_on;
  s->prof_on = false;  // profiling creates events: not here
  int rc = batch_params(s, p, st, seeds, n, LMI_LOC_DEVICE, 0, LMI_MODE_TRAIN, rng_seed, &bp);
  if (rc == LMI_OK) rc = launch_batch_generate(s, pp, &bp, 1, st, false);
  for (int k = 0; rc == LMI_OK && k < s->cfg.hops; ++k) rc = launch_hop(s, pp, 1, st, k, true, true);
  if (rc == LMI_OK) rc = launch_lookup(s, pp, 1, st, 0, s->cfg.hops);
  if (rc == LMI_OK) rc = launch_gather_group(s, pp, 1, st, 0, s->cfg.hops, 0, true);
  if (rc == LMI_OK) {
    hipLaunchKernelGGL(copy_headers_kernel, dim3(1), dim3(64), 0, st, p.st, out->node_counter, out->edge_counter);
    if (hipGetLastError() != hipSuccess) {
      set_error("launch of the header copy failed");
      rc = LMI_ERR_HIP;
    }
  }
  s->prof_on = prof;
  return rc;
}

// What the sticky fault words say, as an error code (no device access, no synchronisation).
static int fault_status(Server *s, int clear) {
  if (!s->fault_host) return LMI_OK;
  const int32_t bad = s->fault_host[kFaultBadId], scan = s->fault_host[kFaultScan];
  if (clear) {
    s->fault_host[kFaultBadId] = s->fault_host[kFaultScan] = 0;
    s->fault_told[kFaultBadId] = s->fault_told[kFaultScan] = false;
  }
  if (scan) LMI_FAIL(LMI_ERR_HIP, "a device scan timed out waiting for an earlier tile: that batch is incomplete");
  if (bad)
    LMI_FAIL(LMI_ERR_BAD_ID, "a seed id outside [0, %lld) was seen on the device and skipped", (long long)s->n_nodes);
  return LMI_OK;
}

int lmi_server_status(lmi_server *h, int clear) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  return fault_status(s, clear);
}

// The same words for lmi_batch_wait: a condition is reported by the first call that sees it and
// not again (lmi_server_status keeps reporting it until it is cleared), so that one bad batch does
// not fail the wait of every good batch after it.
static int fault_status_once(Server *s) {
  if (!s->fault_host) return LMI_OK;
  // one condition per call: when both are pending, the second is told by the next call
  if (s->fault_host[kFaultScan] != 0 && !s->fault_told[kFaultScan]) {
    s->fault_told[kFaultScan] = true;
    LMI_FAIL(LMI_ERR_HIP, "a device scan timed out waiting for an earlier tile: that batch is incomplete");
  }
  if (s->fault_host[kFaultBadId] != 0 && !s->fault_told[kFaultBadId]) {
    s->fault_told[kFaultBadId] = true;
    LMI_FAIL(LMI_ERR_BAD_ID, "a seed id outside [0, %lld) was seen on the device and skipped", (long long)s->n_nodes);
  }
  return LMI_OK;
}

int lmi_batch_wait(lmi_server *h, int pipe, void *stream) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  LMI_TRY(pipe_join(s->pipes[pipe], (hipStream_t)stream));
  return fault_status_once(s);
}

// ------------------------------------------------------------------ outputs
int lmi_batch_view_get(lmi_server *h, int pipe, lmi_batch_view *out) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  if (!out) LMI_FAIL(LMI_ERR_ARG, "null argument");
  Pipe &p = s->pipes[pipe];
  memset(out, 0, sizeof(*out));
  out->ids = p.ids;
  out->features = p.features;
  out->labels = p.labels;
  out->agg_src_ids = p.agg_src_ids;
  out->agg_src_off = p.agg_src_off;
  out->agg_dst_off = p.agg_dst_off;
  out->node_counter = p.st->node_counter;
  out->edge_counter = p.st->edge_counter;
  for (int k = 0; k < LMI_MAX_HOPS; ++k) out->blk_indptr[k] = p.blk_indptr[k];
  out->cache_index = p.cache_index;
  out->max_nodes = s->max_nodes;
  out->max_edges = s->max_edges;
  out->row_bytes = s->row_bytes;
  return LMI_OK;
}

int lmi_batch_counters(lmi_server *h, int pipe, void *stream, int32_t node_counter[16], int32_t edge_counter[16]) {
  Server *s = reinterpret_cast<Server *>(h);
  LMI_TRY(check_pipe(s, pipe));
  DevState hs;
  LMI_TRY(pipe_join(s->pipes[pipe], (hipStream_t)stream));
  LMI_HIP(hipStreamSynchronize((hipStream_t)stream));
  LMI_HIP(hipMemcpy(&hs, s->pipes[pipe].st, sizeof(DevState), hipMemcpyDeviceToHost));
  if (node_counter) memcpy(node_counter, hs.node_counter, 64);
  if (edge_counter) memcpy(edge_counter, hs.edge_counter, 64);
  if (hs.scan_fault) LMI_FAIL(LMI_ERR_HIP, "a device scan timed out waiting for an earlier tile");
  if (hs.bad_id) LMI_FAIL(LMI_ERR_BAD_ID, "a seed id outside [0, %lld) was skipped", (long long)s->n_nodes);
  return LMI_OK;
}

int lmi_idset_batch(lmi_server *h, int mode, int32_t ids_per_batch) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || mode < 0 || mode > 2) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  if (ids_per_batch < 1 || ids_per_batch > s->cfg.batch_size)
    LMI_FAIL(LMI_ERR_CAPACITY, "%d ids per batch outside 1..%d", ids_per_batch, s->cfg.batch_size);
  s->set_batch[mode] = ids_per_batch;
  return LMI_OK;
}

int lmi_steps_per_epoch(lmi_server *h, int mode, int32_t *steps) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !steps || mode < 0 || mode > 2) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  *steps = (int32_t)ceil_div(s->set_n[mode], s->set_batch[mode] ? s->set_batch[mode] : s->cfg.batch_size);
  return LMI_OK;
}

// -------------------------------------------------------------- measurement
int lmi_profile_enable(lmi_server *h, int on) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s) LMI_FAIL(LMI_ERR_ARG, "null server");
  if (on < 0 || on > 2) LMI_FAIL(LMI_ERR_ARG, "profile level must be 0, 1 or 2");
  s->prof_on = on != 0;
  s->prof_level = on;
  s->prof_seq = 0;
  return LMI_OK;
}

int lmi_profile_read(lmi_server *h, lmi_profile *out, int reset) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !out) LMI_FAIL(LMI_ERR_ARG, "null argument");
  LMI_HIP(hipDeviceSynchronize());
  for (auto &e : s->prof_events) {
    float ms = 0.0f;
    if (e.b && hipEventElapsedTime(&ms, e.a, e.b) == hipSuccess) {
      switch (e.kind) {
        case PROF_GATHER_HIT: s->prof.gather_hit_ms += ms; s->prof.gather_hit_launches++; break;
        case PROF_GATHER_MISS: s->prof.gather_miss_ms += ms; s->prof.gather_miss_launches++; break;
        case PROF_SAMPLE: s->prof.sample_ms += ms; s->prof.sample_launches++; break;
        case PROF_LOOKUP: s->prof.lookup_ms += ms; s->prof.lookup_launches++; break;
      }
    } else {
      (void)hipGetLastError();
    }
  }
  for (auto &ev : s->prof_used) s->prof_free.push_back(ev);
  s->prof_used.clear();
  s->prof_open = -1;
  s->prof_events.clear();
  unsigned long long rows[2] = {0, 0};
  LMI_HIP(hipMemcpy(rows, s->d_prof_rows, 16, hipMemcpyDeviceToHost));
  LMI_HIP(hipMemset(s->d_prof_rows, 0, 16));
  s->prof.gather_miss_rows += (int64_t)rows[1];
  if (rows[0] > rows[1]) s->prof.gather_hit_rows += (int64_t)(rows[0] - rows[1]);
  *out = s->prof;
  if (reset) s->prof = lmi_profile{};
  return LMI_OK;
}

int lmi_tune(lmi_server *h, const char *key, int64_t value) {
  Server *s = reinterpret_cast<Server *>(h);
  if (!s || !key) LMI_FAIL(LMI_ERR_ARG, "null argument");
  invalidate_graphs(s);
  if (!strcmp(key, "gather_lanes_per_row")) s->gather_lpr = (int)value;
  else if (!strcmp(key, "gather_unroll")) s->gather_unroll = (int)value;
  else if (!strcmp(key, "gather_vector_bytes")) s->gather_vec = (int)value;
  else if (!strcmp(key, "gather_blocks")) s->gather_blocks = (int)value;
  else if (!strcmp(key, "gather_nontemporal")) s->gather_nt = (int)value;
  else if (!strcmp(key, "gather_adaptive")) s->gather_adaptive = (int)value;
  else if (!strcmp(key, "gather_flat")) s->gather_flat = (int)value;
  else if (!strcmp(key, "miss_flat")) s->miss_flat = (int)value;
  else if (!strcmp(key, "gather_tile_rows")) s->gather_tile_rows = (int)value;
  else if (!strcmp(key, "int8_elements_per_lane")) s->int8_epl = (int)value;
  else if (!strcmp(key, "lds_dedup")) s->lds_dedup = (int)value;
  else if (!strcmp(key, "fuse_count")) s->fuse_count = (int)value;
  else if (!strcmp(key, "protect_hits")) s->protect_hits = (int)value;
  else if (!strcmp(key, "group_miss")) s->group_miss = (int)value;
  else if (!strcmp(key, "lru_early_miss")) s->lru_early_miss = (int)value;
  else if (!strcmp(key, "early_fork")) s->early_fork = (int)value;
  else if (!strcmp(key, "split_lookup")) s->split_lookup = (int)value;
  else if (!strcmp(key, "miss_blocks_early")) s->miss_blocks_early = (int)value;
  else if (!strcmp(key, "table_epochs")) {
    s->table_epochs = std::max<int64_t>(0, value);
    for (auto &p : s->pipes) p.table_dirty = true;
  }
  else if (!strcmp(key, "profile_every")) s->prof_every = (int)std::max<int64_t>(1, value);
  else if (!strcmp(key, "fuse_small_max")) s->fuse_small_max = value;
  else if (!strcmp(key, "split_miss")) s->split_miss = (int)value;
  else if (!strcmp(key, "use_graph")) s->use_graph = (int)value;
  else if (!strcmp(key, "miss_blocks")) s->miss_blocks = (int)value;
  else if (!strcmp(key, "miss_unroll")) s->miss_unroll = (int)value;
  else LMI_FAIL(LMI_ERR_ARG, "unknown tuning key '%s'", key);
  return LMI_OK;
}

// Buffers and events of a measurement, released on every return path.
namespace {
struct BenchScratch {
  void *a = nullptr, *b = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  ~BenchScratch() {
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    if (a) (void)hipFree(a);
    if (b) (void)hipFree(b);
  }
  int events() {
    LMI_HIP(hipEventCreate(&e0));
    LMI_HIP(hipEventCreate(&e1));
    return LMI_OK;
  }
  int elapsed(int repeats, double *ms_out) {
    LMI_HIP(hipEventRecord(e1, 0));
    LMI_HIP(hipEventSynchronize(e1));
    float ms = 0;
    LMI_HIP(hipEventElapsedTime(&ms, e0, e1));
    *ms_out = ms / repeats;
    return LMI_OK;
  }
};
}  // namespace

// Repeats of a measurement kernel go round this many separate copies of its buffers, so that what is
// timed comes from and goes to HBM: a launch repeated on one buffer of a few hundred MB would be
// served in part by the 256 MB memory-side cache in front of HBM, which no gather of a serving loop
// (sixteen output buffer sets, a table of tens of GB) ever is.
static int bench_copies(size_t bytes_per_launch) {
  const size_t want = size_t(3) << 29;  // 1.5 GB of footprint
  return (int)std::max<size_t>(1, std::min<size_t>(64, (want + bytes_per_launch - 1) / std::max<size_t>(bytes_per_launch, 1)));
}

int lmi_bench_host_read(const void *host_ptr, size_t bytes, int repeats, double *ms_per_pass) {
  if (!host_ptr || !ms_per_pass || repeats < 1 || bytes < 16) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  BenchScratch m;
  LMI_HIP(hipMalloc(&m.b, bytes));
  LMI_TRY(m.events());
  const size_t n = bytes / 16;
  hipLaunchKernelGGL(copy_kernel<true>, dim3(1024), dim3(256), 0, 0, (const cp_u32x4 *)host_ptr, (cp_u32x4 *)m.b, n);
  LMI_HIP(hipEventRecord(m.e0, 0));
  for (int r = 0; r < repeats; ++r)
    hipLaunchKernelGGL(copy_kernel<true>, dim3(1024), dim3(256), 0, 0, (const cp_u32x4 *)host_ptr, (cp_u32x4 *)m.b, n);
  LMI_HIP(hipGetLastError());
  return m.elapsed(repeats, ms_per_pass);
}

// Four independent reads per thread at places drawn by a 64-bit mixer; the sum goes nowhere
// unless it hits one particular value, which keeps the loads alive.
static __global__ __launch_bounds__(256) void random_read_kernel(const uint32_t *a, uint64_t n_words, int64_t n_reads,
                                                                uint64_t salt, uint32_t *sink) {
  const int64_t t = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) * 4;
  if (t >= n_reads) return;
  uint32_t v[4];
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    uint64_t x = (uint64_t)(t + k) + salt;
    x ^= x >> 33; x *= 0xff51afd7ed558ccdULL; x ^= x >> 33; x *= 0xc4ceb9fe1a85ec53ULL; x ^= x >> 33;
    v[k] = a[x % n_words];
  }
  const uint32_t acc = v[0] + v[1] + v[2] + v[3];
  if (acc == 0x9E3779B1u) *sink = acc;
}

int lmi_bench_random_read(const void *device_ptr, size_t bytes, int64_t n_reads, int repeats, double *ms_per_pass) {
  if (!device_ptr || !ms_per_pass || repeats < 1 || bytes < 4 || n_reads < 4) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  BenchScratch m;
  LMI_HIP(hipMalloc(&m.a, 4));
  uint32_t *sink = (uint32_t *)m.a;
  LMI_TRY(m.events());
  const int grid = (int)std::min<int64_t>(ceil_div(ceil_div(n_reads, 4), 256), 1 << 30);
  const uint64_t n_words = bytes / 4;
  hipLaunchKernelGGL(random_read_kernel, dim3(grid), dim3(256), 0, 0, (const uint32_t *)device_ptr, n_words, n_reads, 1ull, sink);
  LMI_HIP(hipEventRecord(m.e0, 0));
  for (int r = 0; r < repeats; ++r)
    hipLaunchKernelGGL(random_read_kernel, dim3(grid), dim3(256), 0, 0, (const uint32_t *)device_ptr, n_words, n_reads,
                       (uint64_t)(r + 2) * 0x9E3779B97F4A7C15ull, sink);
  LMI_HIP(hipGetLastError());
  return m.elapsed(repeats, ms_per_pass);
}

int lmi_bench_copy(size_t bytes, int repeats, double *ms_per_copy) {
  if (!ms_per_copy || repeats < 1 || bytes < 16) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  BenchScratch m;
  const int copies = bench_copies(2 * bytes);
  const size_t pitch = (bytes + 255) / 256 * 256;
  LMI_HIP(hipMalloc(&m.a, pitch * copies));
  LMI_HIP(hipMalloc(&m.b, pitch * copies));
  LMI_HIP(hipMemset(m.a, 1, pitch * copies));
  LMI_TRY(m.events());
  const size_t n = bytes / 16;
  auto launch = [&](int r) {
    const size_t at = pitch * (size_t)(r % copies);
    hipLaunchKernelGGL(copy_kernel<false>, dim3(16384), dim3(256), 0, 0, (const cp_u32x4 *)((const char *)m.a + at),
                       (cp_u32x4 *)((char *)m.b + at), n);
  };
  launch(0);
  LMI_HIP(hipEventRecord(m.e0, 0));
  for (int r = 0; r < repeats; ++r) launch(r + 1);
  LMI_HIP(hipGetLastError());
  return m.elapsed(repeats, ms_per_copy);
}

int lmi_bench_copy_launch(size_t bytes, int repeats, double *ms_per_launch) {
  if (!ms_per_launch || repeats < 1 || bytes < 16) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  BenchScratch m;
  const int copies = bench_copies(2 * bytes);
  const size_t pitch = (bytes + 255) / 256 * 256;
  LMI_HIP(hipMalloc(&m.a, pitch * copies));
  LMI_HIP(hipMalloc(&m.b, pitch * copies));
  LMI_HIP(hipMemset(m.a, 1, pitch * copies));
  LMI_TRY(m.events());
  const size_t n = bytes / 16;
  // a grid in proportion to the bytes, as the gathers size theirs, between one block and 64 per compute unit
  const int grid = (int)std::max<size_t>(1, std::min<size_t>(n / (256 * 4), 16384));
  double total = 0.0;
  for (int r = -1; r < repeats; ++r) {  // the first launch warms up and is not counted
    const size_t at = pitch * (size_t)((r + 1) % copies);
    hipExtLaunchKernelGGL(copy_kernel<false>, dim3(grid), dim3(256), 0, 0, m.e0, m.e1, 0,
                          (const cp_u32x4 *)((const char *)m.a + at), (cp_u32x4 *)((char *)m.b + at), n);
    LMI_HIP(hipGetLastError());
    LMI_HIP(hipDeviceSynchronize());
    float ms = 0;
    LMI_HIP(hipEventElapsedTime(&ms, m.e0, m.e1));
    if (r >= 0) total += ms;
  }
  *ms_per_launch = total / repeats;
  return LMI_OK;
}

int lmi_bench_stream(size_t units, int read_bytes, int write_bytes, int misalign, int repeats, int launch_by_launch,
                     double *ms_per_launch) {
  if (!ms_per_launch || repeats < 1 || units < 1) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  const int shape = read_bytes * 100 + write_bytes;
  if (shape != 416 && shape != 816 && shape != 832 && shape != 1616)
    LMI_FAIL(LMI_ERR_ARG, "read : write bytes per unit must be 4:16, 8:16, 8:32 or 16:16");
  if (misalign != 0 && (misalign != 4 || shape != 1616)) LMI_FAIL(LMI_ERR_ARG, "misalign is 0, or 4 with 16:16");
  BenchScratch m;
  const int copies = bench_copies(units * (size_t)(read_bytes + write_bytes));
  const size_t src_pitch = (units * read_bytes + 64 + 255) / 256 * 256, dst_pitch = (units * write_bytes + 64 + 255) / 256 * 256;
  LMI_HIP(hipMalloc(&m.a, src_pitch * copies));
  LMI_HIP(hipMalloc(&m.b, dst_pitch * copies));
  LMI_HIP(hipMemset(m.a, 1, src_pitch * copies));
  LMI_TRY(m.events());
  int turn = 0;
  const int grid = (int)std::max<size_t>(1, std::min<size_t>(units / (256 * 4), 16384));
  auto launch = [&](hipEvent_t e0, hipEvent_t e1) {
    const uint8_t *src = (const uint8_t *)m.a + src_pitch * (size_t)(turn % copies) + misalign;
    uint8_t *dst = (uint8_t *)m.b + dst_pitch * (size_t)(turn % copies) + misalign;
    ++turn;
#define LMI_STREAM(RB_, WB_, A4_)                                                                                   \
  if (e0)                                                                                                           \
    hipExtLaunchKernelGGL((stream_kernel<RB_, WB_, A4_>), dim3(grid), dim3(256), 0, 0, e0, e1, 0, src, dst, units);  \
  else                                                                                                              \
    hipLaunchKernelGGL((stream_kernel<RB_, WB_, A4_>), dim3(grid), dim3(256), 0, 0, src, dst, units)
    if (shape == 416) { LMI_STREAM(4, 16, false); }
    else if (shape == 816) { LMI_STREAM(8, 16, false); }
    else if (shape == 832) { LMI_STREAM(8, 32, false); }
    else if (misalign) { LMI_STREAM(16, 16, true); }
    else { LMI_STREAM(16, 16, false); }
#undef LMI_STREAM
  };
  if (launch_by_launch) {  // each launch alone on the device, timed from its own first to its own last wavefront
    double total = 0.0;
    for (int r = -1; r < repeats; ++r) {
      launch(m.e0, m.e1);
      LMI_HIP(hipGetLastError());
      LMI_HIP(hipDeviceSynchronize());
      float ms = 0;
      LMI_HIP(hipEventElapsedTime(&ms, m.e0, m.e1));
      if (r >= 0) total += ms;
    }
    *ms_per_launch = total / repeats;
    return LMI_OK;
  }
  launch(nullptr, nullptr);
  LMI_HIP(hipEventRecord(m.e0, 0));
  for (int r = 0; r < repeats; ++r) launch(nullptr, nullptr);
  LMI_HIP(hipGetLastError());
  return m.elapsed(repeats, ms_per_launch);
}

int lmi_bench_row_stream(int64_t rows, int64_t src_pitch, int read_bytes, int write_bytes, int64_t table_rows,
                         int repeats, int launch_by_launch, double *ms_per_launch) {
  return lmi_bench_row_stream_shape(rows, src_pitch, read_bytes, write_bytes, table_rows, 0, 0, 0, repeats,
                                    launch_by_launch, ms_per_launch);
}

int lmi_bench_row_stream_shape(int64_t rows, int64_t src_pitch, int read_bytes, int write_bytes, int64_t table_rows,
                               int rows_per_block, int grid_blocks, int every_lane_loads, int repeats,
                               int launch_by_launch, double *ms_per_launch) {
  if (!ms_per_launch || repeats < 1 || rows < 1 || rows > INT32_MAX || table_rows < 2) LMI_FAIL(LMI_ERR_ARG, "bad argument");
  if (rows_per_block < 0 || rows_per_block > 4096 || grid_blocks < 0 || grid_blocks > (1 << 24))
    LMI_FAIL(LMI_ERR_ARG, "a block visit takes 1..4096 rows and a grid has at most 2^24 blocks (0 = chosen here)");
  const int shape = read_bytes * 100 + write_bytes;
  if (shape != 416 && shape != 816 && shape != 1616) LMI_FAIL(LMI_ERR_ARG, "read : write bytes per unit must be 4:16, 8:16 or 16:16");
  if (src_pitch < read_bytes || src_pitch % 4 != 0) LMI_FAIL(LMI_ERR_ARG, "rows are a multiple of 4 bytes and hold a unit");
  const bool a4 = src_pitch % 16 != 0;  // 16-byte accesses that may only assume 4-byte alignment
  if (a4 && shape != 1616) LMI_FAIL(LMI_ERR_ARG, "rows that are no multiple of 16 bytes go with 16:16");
  const int upr = (int)(src_pitch / read_bytes);  // whole units; a row's last few bytes are left out
  if (upr < 1 || upr > (1 << 16)) LMI_FAIL(LMI_ERR_ARG, "row length out of range");  // rows_per_block x upr stays an int
  int lg = 1;
  while ((int64_t(2) << lg) <= table_rows && lg < 31) ++lg;  // the table holds 2^lg rows, at most table_rows
  const int64_t dst_pitch = a4 ? src_pitch : (int64_t)upr * write_bytes;
  BenchScratch m;
  const size_t src_bytes = (size_t)(int64_t(1) << lg) * src_pitch + 64;
  const size_t dst_bytes = ((size_t)rows * dst_pitch + 64 + 255) / 256 * 256;
  const int copies = bench_copies(dst_bytes);  // of the output; the table is as large as the caller says
  LMI_HIP(hipMalloc(&m.a, src_bytes));
  LMI_HIP(hipMalloc(&m.b, dst_bytes * copies));
  LMI_HIP(hipMemset(m.a, 1, src_bytes));
  LMI_TRY(m.events());
  const uint8_t *src = (const uint8_t *)m.a;
  int turn = 0;
  // about 32 KB of output per block visit, at least one row, one block per visit -- unless the caller says otherwise
  const int rpb = rows_per_block > 0 ? rows_per_block
                                     : (int)std::max<int64_t>(1, std::min<int64_t>(64, 32768 / std::max<int64_t>(1, dst_pitch)));
  const int grid = grid_blocks > 0 ? grid_blocks
                                   : (int)std::max<int64_t>(1, std::min<int64_t>((rows + rpb - 1) / rpb, 1 << 20));
  auto launch = [&](hipEvent_t e0, hipEvent_t e1) {
    uint8_t *dst = (uint8_t *)m.b + dst_bytes * (size_t)(turn++ % copies);
#define LMI_ROWS_E(RB_, WB_, A4_, EV_)                                                                                \
  if (e0)                                                                                                            \
    hipExtLaunchKernelGGL((row_stream_kernel<RB_, WB_, A4_, EV_>), dim3(grid), dim3(256), 0, 0, e0, e1, 0, src, dst,  \
                          rows, upr, src_pitch, dst_pitch, lg, rpb);                                                 \
  else                                                                                                               \
    hipLaunchKernelGGL((row_stream_kernel<RB_, WB_, A4_, EV_>), dim3(grid), dim3(256), 0, 0, src, dst, rows, upr,     \
                       src_pitch, dst_pitch, lg, rpb)
#define LMI_ROWS(RB_, WB_, A4_)                               \
  if (every_lane_loads) { LMI_ROWS_E(RB_, WB_, A4_, true); }  \
  else { LMI_ROWS_E(RB_, WB_, A4_, false); }
    if (shape == 416) { LMI_ROWS(4, 16, false) }
    else if (shape == 816) { LMI_ROWS(8, 16, false) }
    else if (a4) { LMI_ROWS(16, 16, true) }
    else { LMI_ROWS(16, 16, false) }
#undef LMI_ROWS
#undef LMI_ROWS_E
  };
  if (launch_by_launch) {
    double total = 0.0;
    for (int r = -1; r < repeats; ++r) {
      launch(m.e0, m.e1);
      LMI_HIP(hipGetLastError());
      LMI_HIP(hipDeviceSynchronize());
      float ms = 0;
      LMI_HIP(hipEventElapsedTime(&ms, m.e0, m.e1));
      if (r >= 0) total += ms;
    }
    *ms_per_launch = total / repeats;
    return LMI_OK;
  }
  launch(nullptr, nullptr);
  LMI_HIP(hipEventRecord(m.e0, 0));
  for (int r = 0; r < repeats; ++r) launch(nullptr, nullptr);
  LMI_HIP(hipGetLastError());
  return m.elapsed(repeats, ms_per_launch);
}

}  // extern "C"
