/*
 * legion_mi.h -- C ABI of the MI355X sampling-server hot path.
 *
 * One opaque server object per GPU.  Batch in: seed node ids.  Batch out:
 * multi-hop sampled blocks (block CSR + the reference's COO view) plus the
 * gathered feature rows, all resident in HBM and described by the reference's
 * two 16-int headers.  Plain pointers and sizes only; every entry point returns
 * 0 on success or a negative LMI_ERR_* code, with text from lmi_last_error().
 *
 * Each declaration names the Legion-IBP interface it stands in for (paths are
 * relative to that tree).  The reference's own `extern "C"` functions take C++
 * object pointers (UnifiedCache*, MemoryPool*, ...) and abort the process on
 * error; here the objects live behind the handle and errors are returned.
 *
 * Threading: a server is not thread-safe; use one server per GPU from one host
 * thread (reference: one std::thread per GPU, engine/server.cu:127-135).  Work
 * is enqueued on the caller's stream and is asynchronous unless stated.
 * `stream` arguments are hipStream_t values passed as void* (NULL = the default
 * stream).  Output buffers are owned by the server and borrowed by the caller
 * until the same pipe is used for another batch (engine/server.cu:337,377).
 * A pipe may be driven from different streams over time: a call that names a pipe
 * orders its stream behind whatever the pipe's previous batch still has queued, on
 * the server's side stream or on the stream that carried that batch -- which must
 * therefore still exist (destroy a stream only after the pipes it drove have been
 * waited for, lmi_batch_wait + lmi_stream_sync, or used from another stream).
 */
#ifndef LEGION_MI_H
#define LEGION_MI_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define LMI_ABI_VERSION 3
#define LMI_MAX_HOPS    3   /* the 16-int headers hold 3 hops (INTRABATCH_CON, include/system_config.cuh:47-57) */
#define LMI_MAX_FANOUT  64  /* one wavefront lane per slot; the reference asserts <= 32 (operator_impl.cu:504) */
#define LMI_MAX_PIPES   16  /* output buffer sets; the reference uses INTERBATCH_CON = 2 */
#define LMI_MAX_GROUP   8   /* mini-batches one lmi_run_group call can issue together */

enum {
  LMI_OK = 0,
  LMI_ERR_ARG = -1,      /* bad argument / wrong call order */
  LMI_ERR_HIP = -2,      /* a HIP runtime call failed */
  LMI_ERR_STATE = -3,    /* required object (graph, features, cache) not loaded */
  LMI_ERR_CAPACITY = -4, /* request exceeds configured capacity */
  LMI_ERR_BAD_ID = -5    /* a seed id outside [0, n_nodes) was seen on the device */
};

enum { LMI_F32 = 0, LMI_F16 = 1 };                       /* feature element type */
enum { LMI_LOC_HOST = 0, LMI_LOC_DEVICE = 1 };           /* where an input pointer lives */
enum { LMI_MODE_TRAIN = 0, LMI_MODE_VALID = 1, LMI_MODE_TEST = 2 }; /* TRAINMODE.. (include/system_config.cuh) */
/* id->slot table layout of the static / int8 caches: open-addressing hash (8 B per
 * slot, load <= 0.5), direct map (4 B per node), or membership bitmap with a
 * running rank (16 B per 64 nodes; slot = rank of the node among cached nodes) */
enum { LMI_TABLE_HASH = 0, LMI_TABLE_DIRECT = 1, LMI_TABLE_RANK = 2 };
/* how the static / int8 hot set is ranked: by out-degree, or by how often presampling
 * touched a node (the reference's policy, cache/cache.cu:354-447); ties by ascending id */
enum { LMI_POLICY_DEGREE = 0, LMI_POLICY_PRESAMPLED = 1 };
enum { LMI_CACHE_NONE = 0, LMI_CACHE_STATIC = 1, LMI_CACHE_LRU = 2, LMI_CACHE_INT8 = 3 };

typedef struct lmi_server lmi_server;

/* Replaces the positional ./meta_config line + argv of the reference
 * (storage/storage_management.cu:33-104, main.cu:9-14). */
typedef struct lmi_config {
  int32_t  device_id;
  int32_t  batch_size;              /* max seeds per batch */
  int32_t  hops;                    /* 1..LMI_MAX_HOPS */
  int32_t  fanout[LMI_MAX_HOPS];    /* per hop, 1..LMI_MAX_FANOUT */
  int32_t  feat_dim;                /* elements per feature row */
  int32_t  feat_dtype;              /* LMI_F32 | LMI_F16 */
  int32_t  pipes;                   /* 1..LMI_MAX_PIPES output buffer sets */
  int32_t  reserved;
  uint64_t seed;                    /* default RNG seed (per-batch seeds may override) */
} lmi_config;

/* Device pointers of one pipe's outputs: the reference's per-pipe MemoryPool /
 * IPC buffers (engine/memorypool.cuh:20-221, engine/ipc_service.cu:140-206) plus
 * the block-CSR row pointers.  Row i of `features` belongs to ids[i].  Edges of
 * hop k (1-based) are agg_*[edge_counter[12+k] .. +edge_counter[9+k]) in local
 * ids; block k has node_counter[9+k] sources and node_counter[9+k-1]
 * destinations (training_backend/ipc_service.cpp:61-68). */
typedef struct lmi_batch_view {
  int32_t *ids;                       /* [max_nodes] global ids, local-id order */
  void    *features;                  /* [max_nodes][feat_dim] feat_dtype */
  int32_t *labels;                    /* [batch_size] (-1 when no labels loaded) */
  int32_t *agg_src_ids;               /* [max_edges] sampled neighbours, global ids */
  int32_t *agg_src_off;               /* [max_edges] COO source, local ids */
  int32_t *agg_dst_off;               /* [max_edges] COO destination, local ids */
  int32_t *node_counter;              /* [16] */
  int32_t *edge_counter;              /* [16] */
  int32_t *blk_indptr[LMI_MAX_HOPS];  /* hop k: [n_{k-1}+1] row pointers into hop k's edge segment */
  int32_t *cache_index;               /* [max_nodes] cache slot per row, -1 = miss */
  int64_t  max_nodes, max_edges;
  int64_t  row_bytes;                 /* bytes of one row of `features` (filled by lmi_batch_view_get) */
} lmi_batch_view;

typedef struct lmi_cache_info {
  int32_t kind;                /* LMI_CACHE_* */
  int32_t table_kind;          /* LMI_TABLE_* (static / int8) */
  int64_t capacity_rows;
  int64_t row_bytes;           /* bytes of one cached row */
  int64_t table_bytes;         /* id->slot table footprint */
  int64_t n_sets; int32_t ways; int32_t lru_tick;
} lmi_cache_info;

/* Per-kernel device time, measured with HIP events on the launching stream. */
typedef struct lmi_profile {
  double  gather_hit_ms;   int64_t gather_hit_launches;  int64_t gather_hit_rows;
  double  gather_miss_ms;  int64_t gather_miss_launches; int64_t gather_miss_rows;
  double  sample_ms;       int64_t sample_launches;      /* all kernels of the sampling hops */
  double  lookup_ms;       int64_t lookup_launches;
  double  batch_ms;        int64_t batches;              /* batch_ms reserved (0); batches = mini-batches the profiled calls served */
} lmi_profile;

/* ---- lifecycle ------------------------------------------------------- */
int         lmi_abi_version(void);
const char *lmi_last_error(void);                               /* thread-local text */
/* Server::Initialize + Runner::Initialize (engine/server.cu:48-92,178-301) */
int lmi_server_create(const lmi_config *cfg, lmi_server **out);
/* Server::Finalize / Runner::Finalize (engine/server.cu:137-170,402-451) */
int lmi_server_destroy(lmi_server *s);
/* Adds output buffer sets until the server has `pipes` of them (1..LMI_MAX_PIPES; never removes
 * one, so views of the existing sets stay valid).  The reference fixes INTERBATCH_CON = 2 at compile
 * time (include/system_config.cuh:47-57); a runner that issues groups of batches wants two groups'
 * worth.  Allocates device memory: not inside a batch loop. */
int lmi_server_pipes(lmi_server *s, int32_t pipes);

/* ---- memory helpers (engine/server_imp.cuh:2-52) ---------------------- */
int lmi_host_alloc(size_t bytes, void **host_ptr);             /* host_alloc_space: pinned + mapped */
int lmi_host_free(void *host_ptr);
int lmi_device_alloc(size_t bytes, void **dev_ptr);            /* d_alloc_space */
int lmi_device_free(void *dev_ptr);                            /* d_free_space */
int lmi_copy_to_host(void *host_dst, const void *dev_src, size_t bytes);   /* d_copy_2_h (synchronous) */
int lmi_copy_to_device(void *dev_dst, const void *host_src, size_t bytes); /* synchronous */
/* Asynchronous device-to-device copy on `stream`. */
int lmi_copy_device(void *dev_dst, const void *dev_src, size_t bytes, void *stream);
/* Memory shared with another process: what the reference does with cudaIpcGetMemHandle on the
 * sampler side (engine/ipc_service.cu:163-192) and cudaIpcOpenMemHandle on the trainer side
 * (training_backend/ipc_cuda_kernel.cu:35-173).  lmi_ipc_export fills the 64-byte handle of the
 * allocation that holds dev_ptr and says where in it dev_ptr lies and how large it is; an
 * allocation of LMI_IPC_MAX_BYTES or more is refused (LMI_ERR_CAPACITY): split it.  The
 * importing process calls lmi_ipc_open once per distinct handle, adds the offset, and closes
 * the mapping with lmi_ipc_close before it exits. */
#define LMI_IPC_HANDLE_BYTES 64
#define LMI_IPC_MAX_BYTES    ((int64_t)1 << 31)
int lmi_ipc_export(const void *dev_ptr, void *handle, int64_t *offset, int64_t *alloc_bytes);
int lmi_ipc_open(const void *handle, void **dev_base);
int lmi_ipc_close(void *dev_base);
int lmi_stream_create(void **stream);
int lmi_stream_destroy(void *stream);
int lmi_stream_sync(void *stream);
int lmi_device_sync(void);

/* ---- storage ---------------------------------------------------------- */
/* GraphStorage::Build (storage/graph_storage.cu:12-73): CSR with int64 row
 * pointers and int32 neighbour ids.  LMI_LOC_HOST copies into HBM;
 * LMI_LOC_DEVICE borrows caller-owned HBM (must outlive the server). */
int lmi_graph_load(lmi_server *s, const int64_t *indptr, const int32_t *indices,
                   int64_t n_nodes, int64_t n_edges, int location);
/* FeatureStorage::Build (storage/feature_storage.cu:18-90): row-major table,
 * row v = features of node v.  LMI_LOC_HOST must come from lmi_host_alloc and is
 * read zero-copy by the device on cache misses; LMI_LOC_DEVICE = table in HBM. */
int lmi_features_attach(lmi_server *s, const void *rows, int64_t n_rows, int location);
/* Training / validation / testing id sets and labels (storage_management.cu:124-279);
 * labels may be NULL.  Always copied into HBM. */
int lmi_idset_load(lmi_server *s, int mode, const int32_t *ids, const int32_t *labels,
                   int64_t n, int location);
/* Ids per batch of id set `mode` when batches are sliced from the set (1 .. batch_size;
 * default batch_size).  The reference serves validation and test batches of their own
 * size (GetCurrentBatchsize, engine/ipc_service.cu:228-236). */
int lmi_idset_batch(lmi_server *s, int mode, int32_t ids_per_batch);

/* ---- presampling (GPUServer::PreSc + PreSCCacheController, engine/server.cu:94-122,
 *      cache/cache.cu:43-71) ------------------------------------------------------ */
/* Samples batches first_batch .. first_batch+n_batches-1 of id set `mode` (no lookup, no
 * gather) and adds one count per sampled id to the per-node hotness table.  Enqueued on
 * `stream`; RNG seeds are the default per-batch seeds, so the same batches are served later. */
int lmi_presample(lmi_server *s, int pipe, void *stream, int mode, int32_t first_batch, int32_t n_batches);
/* HotnessMeasure for the batch currently in `pipe` (what IOComplete does while presampling,
 * engine/operator_impl.cu:607-636). */
int lmi_op_hotness(lmi_server *s, int pipe, void *stream);
int lmi_presample_reset(lmi_server *s);                      /* forget the counts */
int lmi_hotness_dump(lmi_server *s, uint32_t *counts, int64_t n);   /* synchronous read-back */
/* Ranking used by the next lmi_cache_build_static / lmi_cache_build_int8. */
int lmi_cache_policy(lmi_server *s, int policy);

/* ---- caches (UnifiedCache::FillUp, cache/cache.cu:559-656) -------------- */
/* Static hot-set cache: the capacity_rows nodes ranked first by (key descending, id
 * ascending); key = out-degree, or the presampling count under LMI_POLICY_PRESAMPLED. */
int lmi_cache_build_static(lmi_server *s, int64_t capacity_rows, int table_kind);
/* LRU dynamic cache, set-associative (comp_cache/static_cache.cu:20-113), starts empty. */
int lmi_cache_build_lru(lmi_server *s, int64_t n_sets, int32_t ways);
/* Compressed cache: int8 rows + per-row fp32 scale, dequantised in the gather
 * (stands in for StaticCache::insert_features_compressed, static_cache.cu:498-612). */
int lmi_cache_build_int8(lmi_server *s, int64_t capacity_rows, int table_kind);
int lmi_cache_info_get(lmi_server *s, lmi_cache_info *out);
/* Test/diagnostic read-back: slot of every node (-1 = not cached), synchronous.
 * For the LRU cache `aux` (may be NULL) receives last_use per slot and slot_of is
 * indexed by slot and receives the key stored there. */
int lmi_cache_dump(lmi_server *s, int32_t *slot_of, int64_t n, int32_t *aux);

/* ---- operators (engine/operator_impl.cuh:11-69, engine/operator.h:27-35) -- */
/* BatchGenerate: stage the seeds as local ids 0..n-1.  seeds == NULL takes slice
 * `batch_counter` of the id set `mode` (batch_generate, operator_impl.cu:28-56);
 * otherwise `n` caller seeds at `seeds_location`.  rng_seed 0 = cfg.seed + batch_counter. */
int lmi_op_batch_generate(lmi_server *s, int pipe, void *stream, const int32_t *seeds, int32_t n,
                          int seeds_location, int32_t batch_counter, int mode, uint64_t rng_seed);
/* RandomSample for hop `hop` (0-based): sample, dedup, relabel, update headers
 * (random_sample + construct_graph + counter_update, operator_impl.cu:178-317,440-553). */
int lmi_op_random_sample(lmi_server *s, int pipe, void *stream, int hop);
/* FeatureCacheLookup for segment `segment`: 0 = seeds, k = nodes added by hop k
 * (FindFeat + FeatCacheLookup, cache/cache.cu:314-338,743-803). */
int lmi_op_cache_lookup(lmi_server *s, int pipe, void *stream, int segment);
/* IOSubmit: empty in the reference too (operator_impl.cu:578-595). */
int lmi_op_io_submit(lmi_server *s, int pipe, void *stream);
/* IOComplete (operator_impl.cu:607-636): end of batch; inserts this batch's
 * misses into the LRU cache. */
int lmi_op_io_complete(lmi_server *s, int pipe, void *stream);
/* Runner::RunOnce (engine/server.cu:330-400): the whole operator chain with one
 * gather over all rows.  With lmi_tune("use_graph", 1) and a non-default stream the
 * sampling part replays a HIP graph captured on first use instead of launching its
 * kernels one by one.  Returns with the host-link part of the gather
 * possibly still running on the server's side stream: see lmi_batch_wait. */
int lmi_run_once(lmi_server *s, int pipe, void *stream, const int32_t *seeds, int32_t n,
                 int seeds_location, int32_t batch_counter, int mode, uint64_t rng_seed);

/* n_batches <= LMI_MAX_GROUP mini-batches at once, batch k into pipe pipes[k] (distinct pipes): the same as
 * n_batches calls of lmi_run_once, but every launch of the sampling phase serves all of them
 * (those kernels are latency-bound, so the batches after the first cost little).  seeds,
 * n_seeds and rng_seeds may be NULL (slices batch_counters[k] of id set `mode`, default RNG
 * seeds).  Not with the LRU cache, whose state advances batch by batch.  No counterpart in
 * the reference, which runs one batch per RunOnce. */
int lmi_run_group(lmi_server *s, int n_batches, const int32_t *pipes, void *stream,
                  const int32_t *const *seeds, const int32_t *n_seeds, int seeds_location,
                  const int32_t *batch_counters, int mode, const uint64_t *rng_seeds);

/* ---- one batch without any allocation ---------------------------------- */
/* Limits of lmi_run_once_static: the server's worst-case rows per batch (max_nodes of its
 * batch view) and worst-case edges of its largest hop, e.g. batch 800 with fan-out [25, 10]. */
#define LMI_STATIC_MAX_NODES      (1 << 18)
#define LMI_STATIC_MAX_HOP_EDGES  (1 << 18)
/* bytes of device memory the library holds per GPU for it, from load to process end */
#define LMI_STATIC_SCRATCH_BYTES  ((size_t)10 << 20)
/* No counterpart in the reference.  For callers that cannot allocate device memory: code under
 * HIP graph capture, tight serving loops, harnesses that forbid it.  The same batch as
 * lmi_run_once (all hops, one lookup, one gather over all rows; hits and misses both on
 * `stream`, no side stream, nothing left pending), but every output goes into buffers the CALLER
 * owns -- `out` names them, all device memory, sized for the server's worst case:
 * ids / cache_index [max_nodes], features [max_nodes][feat_dim], labels [batch_size],
 * agg_* [max_edges], blk_indptr[k] [n_k + 1], node_counter / edge_counter [16] -- and the
 * kernels' scratch (dedup table, per-edge slots, scan status words, miss list, batch state)
 * lives in one file-scope device array of LMI_STATIC_SCRATCH_BYTES per GPU instead of a pipe.
 * Calls no hipMalloc / hipFree and nothing else that allocates.  `seeds` is device memory.
 * Servers whose worst case exceeds the limits above, and servers with the LRU cache (whose
 * insertion needs per-pipe state), get LMI_ERR_CAPACITY / LMI_ERR_STATE.  Every call on a GPU
 * shares that GPU's array: calls that overlap on one GPU (two streams, two threads, two
 * servers) race; calls that follow each other on one stream do not.  What a call launches
 * depends on nothing but its arguments and the device memory they name (the dedup table in the
 * scratch is wiped by every call): captured in a HIP graph, it may be replayed, with new
 * seeds written into the same `seeds` buffer between replays. */
int lmi_run_once_static(lmi_server *s, void *stream, const int32_t *seeds, int32_t n,
                        uint64_t rng_seed, const lmi_batch_view *out);

/* ---- outputs ----------------------------------------------------------- */
/* Makes `stream` wait until every output of the pipe's last batch is complete,
 * including rows still being fetched over the host link on the server's own side
 * stream.  This is the point where the reference's runner has seen its last
 * operator's event and posts the batch (engine/server.cu:356-361,377).  Any other
 * call on the same pipe waits in the same way first. */
int lmi_batch_wait(lmi_server *s, int pipe, void *stream);
/* What the reference answers with printf + exit(EXIT_FAILURE) (cudaCheckError,
 * engine/memorypool.cuh:9-17; soft failures operator_impl.cu:144-151): a condition raised
 * by a kernel of ANY batch since the server was created (or since the last call with
 * clear != 0) -- a seed id outside [0, n_nodes) (LMI_ERR_BAD_ID; the id was skipped) or a
 * device scan that gave up waiting (LMI_ERR_HIP; that batch is incomplete).  The kernels
 * record it in pinned host memory, so this call reads no device memory and synchronises
 * nothing; a condition of a batch still running shows once that batch is done.  It keeps
 * reporting the condition until a call with clear != 0 (which reports it one last time).
 * lmi_batch_wait returns the same code, but only ONCE per condition (to the first wait that
 * sees it; again after a clear): one bad batch does not fail the wait of every good batch
 * after it.  Neither call says WHICH batch: the words are read as the host sees them, so the
 * wait of the faulty batch itself can still pass and a later one report.  A per-batch verdict
 * is what lmi_batch_counters gives (it synchronises and reads the batch's own flags). */
int lmi_server_status(lmi_server *s, int clear);
int lmi_batch_view_get(lmi_server *s, int pipe, lmi_batch_view *out);
/* Synchronises `stream`, copies both headers to the host, reports a bad seed id. */
int lmi_batch_counters(lmi_server *s, int pipe, void *stream, int32_t node_counter[16],
                       int32_t edge_counter[16]);
/* Batches an id set holds: ceil(size / ids per batch).  The reference's own step counts
 * (Coordinate, engine/ipc_service.cu:60-128: it drops the training set's last batch)
 * are computed by the host layer above this ABI. */
int lmi_steps_per_epoch(lmi_server *s, int mode, int32_t *steps);

/* ---- measurement ------------------------------------------------------- */
/* level 0: off; 1: HIP events bracket the sampling phase and the lookup of a batch and each
 * gather kernel carries a start / stop event pair of its own; 2: only the gather kernels
 * are timed, nothing is queued between kernels.  Rows per gather are counted on the device
 * for the same batches.  lmi_tune("profile_every", n) profiles one batch in n. */
int lmi_profile_enable(lmi_server *s, int level);
int lmi_profile_read(lmi_server *s, lmi_profile *out, int reset);  /* synchronises the device */
/* Tuning knobs by name (e.g. "gather_lanes_per_row", "gather_unroll", "lds_dedup"). */
int lmi_tune(lmi_server *s, const char *key, int64_t value);
/* Plain device copy of `bytes` bytes, repeated; returns mean ms per copy
 * (the measured HBM ceiling quoted beside the nominal peak). */
int lmi_bench_copy(size_t bytes, int repeats, double *ms_per_copy);
/* The same copy timed launch by launch: every launch starts on an idle device and is timed from
 * its own first to its own last wavefront (the start / stop events of the launch itself), which
 * is how the gather kernels are timed.  What a launch of this size can reach at all: a launch of
 * a few hundred MB spends a visible part of its time filling and draining the device. */
int lmi_bench_copy_launch(size_t bytes, int repeats, double *ms_per_launch);
/* The ceiling of a gather's SHAPE: a streaming kernel that reads read_bytes and writes write_bytes
 * per lane and step -- 4:16 (int8 -> fp32), 8:16 (int8 -> fp16), 8:32, or 16:16 (a row mover; with
 * misalign = 4 both sides sit 4 bytes off a 16-byte boundary, as rows of 16 k + 12 bytes do) --
 * over `units` such steps, contiguous, no indirection.  launch_by_launch != 0 times every launch
 * alone, from its own first to its own last wavefront (lmi_bench_copy_launch); 0 times `repeats`
 * launches back to back (lmi_bench_copy).  A 1:1 copy says little about a kernel that writes twice
 * what it reads: HBM takes writes more slowly than reads. */
int lmi_bench_stream(size_t units, int read_bytes, int write_bytes, int misalign, int repeats, int launch_by_launch,
                     double *ms_per_launch);
/* The same with the one property of a gather that lmi_bench_stream leaves out: the rows come from all
 * over a large table.  Output row r (rows contiguous) is row hash(r) of a table of the largest power
 * of two <= table_rows rows, src_pitch bytes each, moved as units of read_bytes in and write_bytes
 * out (4:16, 8:16, 16:16; a pitch that is no multiple of 16 goes with 16:16 and 16-byte accesses at
 * 4-byte alignment).  The source row is computed, not loaded: no index to wait for, no table
 * lookup, no LDS, no barrier.  What is left between a gather and this figure is the gather's own
 * doing; what is left between this figure and lmi_bench_stream is what HBM charges for rows that
 * do not follow each other. */
int lmi_bench_row_stream(int64_t rows, int64_t src_pitch, int read_bytes, int write_bytes, int64_t table_rows,
                         int repeats, int launch_by_launch, double *ms_per_launch);
/* The same kernel with the launch shape in the caller's hands, for studying what a gather's own choices
 * cost: rows_per_block (0 = about 32 KB of output per block visit), grid_blocks (0 = one block per
 * visit; more = blocks that find nothing to do and leave, as a grid sized for the worst case of a
 * batch holds; fewer = blocks that loop), every_lane_loads != 0 (lanes without a unit in a block's
 * last pass issue their loads anyway and only skip the store).  Refused: more than 4096 rows per
 * visit, more than 2^24 blocks, rows of more than 2^16 units, more than 2^31 - 1 rows. */
int lmi_bench_row_stream_shape(int64_t rows, int64_t src_pitch, int read_bytes, int write_bytes, int64_t table_rows,
                               int rows_per_block, int grid_blocks, int every_lane_loads, int repeats,
                               int launch_by_launch, double *ms_per_launch);
/* Streaming zero-copy read of `bytes` bytes of pinned host memory (from lmi_host_alloc) into
 * HBM, repeated; returns mean ms per pass (the measured host-link ceiling). */
int lmi_bench_host_read(const void *host_ptr, size_t bytes, int repeats, double *ms_per_pass);
/* n_reads independent 4-byte reads at pseudo-random places of a device array of `bytes` bytes
 * (e.g. the neighbour array), repeated; returns mean ms per pass: the rate of cold random reads
 * this device sustains, which is what bounds the sampling kernels. */
int lmi_bench_random_read(const void *device_ptr, size_t bytes, int64_t n_reads, int repeats, double *ms_per_pass);

/* ---- synthetic inputs (stand-in for the reference's dataset tooling) ---- */
/* Power-law graph generated in HBM: degree(v) by inverse-CDF lookup of a Philox
 * word in `cdf` (host array of uint32 thresholds), neighbours uniform (mode 0) or
 * degree-proportional (mode 1).  The caller owns the returned device arrays. */
int lmi_synth_graph(uint64_t seed, const uint32_t *cdf, int32_t cdf_len, int64_t n_nodes,
                    int32_t mode, int64_t **d_indptr, int32_t **d_indices, int64_t *n_edges);
int lmi_synth_trainset(uint64_t seed, int64_t n_nodes, int32_t n_train, int32_t *host_ids);
/* N(0,1) rows written straight into (pinned) host or device memory by the GPU. */
int lmi_synth_features(uint64_t seed, void *rows, int64_t n_rows, int32_t dim, int32_t dtype);

#ifdef __cplusplus
}
#endif
#endif /* LEGION_MI_H */
