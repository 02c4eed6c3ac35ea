// Host-side C++ interface of the sampling server, above the C ABI.
//
// Same class and factory names, argument meaning and call order as the
// reference's host interface, so its callers keep compiling against this header:
//   Server / Runner / RunnerParams / NewGPUServer / NewGPURunner
//       (Legion-IBP sampling_server/src/engine/server.h:5-34; callers main.cu:8-16,
//        sampling_server.cpp:9-13)
//   Operator / OpParams / New*OP factories
//       (sampling_server/src/engine/operator.h:6-35)
// Everything below these classes goes through include/legion_mi.h; no HIP type
// appears here (streams and events travel as void*).
//
// Differences a caller can observe:
//   * one GPU: Initialize() rejects global_shard_count != 1 and PreSc() rejects a
//     cache aggregation mode other than 0 (no cross-GPU cache pooling);
//   * errors are printed and end the process, like the reference's cudaCheckError,
//     but every message names the failing C-ABI call and its error text;
//   * `dyn_cache` keeps the reference's bit meaning where a counterpart exists:
//     0 = static hot-set cache, DYN_ENABLE (1) = LRU dynamic cache,
//     DYN_COMP (8) = compressed (int8) cache; other bits are ignored;
//   * Run() serves the reference's schedule (per epoch the training steps, then the
//     validation steps; the test steps after the last epoch; engine/server.cu:124-135,
//     engine/ipc_service.cu:60-128,212-260);
//   * the hand-off to a trainer is a callback (SetBatchSink) and, once EnableHandoff(true)
//     was called, the reference's shared-memory slab + two named semaphores per output
//     buffer set (ipc_service.hpp) towards a trainer in another process, or on another thread
//     of this one; the buffers either receives are the reference's output contract;
//   * Run() issues the schedule in groups of up to LMI_MAX_GROUP batches of one mode, on twice
//     as many output buffer sets, unless the batches are taken one by one (the trainer's two
//     buffer sets, the LRU cache, the operator table, LEGION_MI_GROUP=1); a sink then sees a
//     group's batches, in order, once the next group has been issued.
#pragma once

#include <cstdint>
#include <string>
#include <vector>

#include "../../include/legion_mi.h"

// dyn_cache bits understood here (reference: comp_cache/cache_helper.cuh:34-45)
enum LegionDynFlags : int { LEGION_DYN_ENABLE = 1 << 0, LEGION_DYN_COMP = 1 << 3 };

struct RunnerParams {
  int device_id;
  std::vector<int> fanout;
  void *cache;    // unused: the caches live behind the lmi_server handle
  void *graph;    // unused
  void *feature;  // unused
  void *env;      // lmi_server* of this GPU
  int global_batch_id;
  bool in_memory;
  int dyn_cache;
  // additions (defaulted, so reference-style aggregate use still works)
  bool fused = false;  // true: RunOnce calls lmi_run_once instead of the operator table
  int mode = LMI_MODE_TRAIN;
  int feature_dim = 0;
  void *ipc = nullptr;  // IPCEnv* (ipc_service.hpp; the reference passes it in `env`).  When set,
                        // global_batch_id counts over the whole schedule and the mode and the
                        // batch's place in its id set come from it; when null, global_batch_id
                        // is the place in id set `mode`.
  bool defer_join = false;  // true: RunOnce does not order the stream behind the batch's host-link
                            // gather (nobody reads the batch yet); the pipe's next batch does, so the
                            // gather overlaps the sampling of the batch in between
  bool defer_post = false;  // hand-off only.  false: RunOnce returns with its batch posted to the trainer,
                            // as the reference's does.  true: it returns with the batch BEFORE posted and
                            // its own still running; the next RunOnce, Flush or Finalize posts that one
  int pipes = 2;            // output buffer sets RunGroup takes in turn (lmi_server_pipes made them)
};

// Called once per finished batch with the pipe's device buffers; the stream has
// been made to wait for the whole batch (lmi_batch_wait) before the call.
typedef void (*LegionBatchSink)(const lmi_batch_view *batch, int device_id, int pipe, void *stream, void *user);

class Server {
 public:
  virtual ~Server() {}
  // Reads ./meta_config and the dataset it names, creates the per-GPU server.
  virtual void Initialize(int global_shard_count, std::vector<int> fanout, int in_memory_mode, int dyn_cache) = 0;
  // Builds the feature cache: ranked by degree, or (LEGION_MI_PRESAMPLE set) by one presampling
  // pass over the training set, which is what the reference does here.
  virtual void PreSc(int cache_agg_mode) = 0;
  // epoch x steps mini-batches through the runner.
  virtual void Run() = 0;
  virtual void Finalize() = 0;
  // additions
  virtual void SetBatchSink(LegionBatchSink sink, void *user) = 0;
  // Before Initialize: serve batches through the semaphore handshake of ipc_service.hpp,
  // waiting at most wait_seconds for the trainer to release a buffer set.
  virtual void EnableHandoff(bool on, double wait_seconds) = 0;
  virtual lmi_server *Handle(int device_id) = 0;
};
Server *NewGPUServer();

class Runner {
 public:
  virtual ~Runner() {}
  virtual void Initialize(RunnerParams *params) = 0;
  virtual void InitializeFeaturesBuffer(RunnerParams *params) = 0;  // buffers are sized at create: no-op
  virtual void RunPreSc(RunnerParams *params) = 0;                  // sampling only, no gather
  virtual void RunOnce(RunnerParams *params) = 0;
  virtual void Finalize(RunnerParams *params) = 0;
  // additions
  // `count` <= LMI_MAX_GROUP consecutive batches of one mode, the first params->global_batch_id,
  // every launch shared by all of them (lmi_run_group), into `count` of the params->pipes buffer
  // sets taken in turn; pipes_out (may be null) receives the set of each batch.  No hand-off.
  virtual void RunGroup(RunnerParams *params, int count, int *pipes_out) = 0;
  virtual void Flush(RunnerParams *params) = 0;  // posts the batch a RunOnce with defer_post left behind
  virtual int CurrentPipe() const = 0;  // pipe holding the batch issued last
  virtual void *Stream() const = 0;
};
Runner *NewGPURunner();

struct OpParams {
  int device_id;
  void *stream;  // hipStream_t
  void *event;   // hipEvent_t (unused: ordering is by stream)
  void *memorypool;  // unused
  void *cache;       // unused
  void *graph;       // unused
  void *feature;     // unused
  void *env;         // lmi_server*
  int neighbor_count;  // fanout of the hop this operator samples
  bool is_presc;
  bool in_memory;
  int hop_num;
  int dyn_cache;
  // additions
  int pipe = 0;
  int global_batch_id = 0;
  int mode = LMI_MODE_TRAIN;
};

class Operator {
 public:
  virtual ~Operator() {}
  virtual void run(OpParams *params) = 0;
};

// op_id is the slot in the runner's table, as in the reference: slot 0 stages the
// seeds, slots 3k sample hop k, slots 3k+1 look up and gather, slots 3k+2 are the
// (empty) IO submit, the last slot completes the batch (engine/server.cu:218-228).
Operator *NewBatchGenerateOP(int op_id);
Operator *NewRandomSampleOP(int op_id);
Operator *NewCacheLookupOP(int op_id);
Operator *NewSSDIOSubmitOP(int op_id);
Operator *NewSSDIOCompleteOP(int op_id);

// The one-line ./meta_config the reference's launcher writes
// (legion_server.py:43-44; parsed positionally in storage_management.cu:33-104).
struct LegionMetaConfig {
  std::string dataset_path;
  int batch_size = 0;
  int64_t node_num = 0, edge_num = 0;
  int feature_dim = 0;
  int64_t training_set_num = 0, validation_set_num = 0, testing_set_num = 0;
  int64_t cache_memory = 0;  // bytes
  int epoch = 1;
  std::string feature_path;  // optional alternative directory for features / labels
};
bool LegionReadMetaConfig(const std::string &path, LegionMetaConfig *out, std::string *error);

// A sampling server on a thread of the calling process, for a trainer that lives in the
// same process (trainer_ipc.hpp): Initialize + PreSc run before the call returns, Run and
// Finalize go on in the background.  The meta config is ./meta_config, or the file the
// environment variable LEGION_MI_META_CONFIG names.  One server per process at a time.
extern "C" int legion_server_start(int gpu_number, int cache_agg_mode, int dyn_cache, const int32_t *fanout,
                                   int hops, int handoff, double wait_seconds);
extern "C" int legion_server_join(void);  // waits for Run + Finalize; 0, or -1 if none was started
