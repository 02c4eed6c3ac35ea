// Host shim: the reference's Server / Runner / Operator classes on top of the C ABI.
// Plain C++17, no HIP headers: every device interaction is an lmi_* call.
//
// Reference behaviour followed here (Legion-IBP sampling_server/src):
//   engine/server.cu:48-170     GPUServer: Initialize -> PreSc -> Run -> Finalize
//   engine/server.cu:178-400    GPURunner: operator table, two output buffer sets
//   engine/operator.cu:10-150   operator classes forwarding to the extern "C" layer
//   storage/storage_management.cu:33-279   ./meta_config + dataset files
#include "legion_host.hpp"
#include "ipc_service.hpp"

#include <sys/mman.h>
#include <sys/stat.h>
#include <fcntl.h>
#include <unistd.h>

#include <chrono>
#include <condition_variable>
#include <mutex>
#include <thread>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iostream>
#include <sstream>

namespace {

[[noreturn]] void die(const char *what) {
  std::fprintf(stderr, "legion_mi failure in %s: %s\n", what, lmi_last_error());
  std::exit(EXIT_FAILURE);
}
#define LMI_MUST(call)                 \
  do {                                 \
    if ((call) != LMI_OK) die(#call);  \
  } while (0)

// Reads a whole binary file into `dst` (at most `bytes`); returns bytes read or -1.
// The reference mmaps and never unmaps (storage_management_impl.cuh:48-123); a
// buffered read into the final buffer does the same job without the leak.
int64_t read_file(const std::string &path, void *dst, int64_t bytes) {
  const int fd = open(path.c_str(), O_RDONLY);
  if (fd < 0) return -1;
  int64_t done = 0;
  while (done < bytes) {
    const ssize_t r = read(fd, (char *)dst + done, (size_t)std::min<int64_t>(bytes - done, int64_t(1) << 30));
    if (r <= 0) break;
    done += r;
  }
  close(fd);
  return done;
}

void must_read(const std::string &path, void *dst, int64_t bytes) {
  const int64_t got = read_file(path, dst, bytes);
  if (got != bytes) {
    std::fprintf(stderr, "cannot read %lld bytes from %s (got %lld)\n", (long long)bytes, path.c_str(), (long long)got);
    std::exit(EXIT_FAILURE);
  }
}

// ---------------------------------------------------------------- operators
class BatchGenerateOP : public Operator {
 public:
  explicit BatchGenerateOP(int id) : op_id_(id) {}
  void run(OpParams *p) override {
    LMI_MUST(lmi_op_batch_generate((lmi_server *)p->env, p->pipe, p->stream, nullptr, 0, LMI_LOC_DEVICE,
                                   p->global_batch_id, p->mode, 0));
  }
 private:
  int op_id_;
};

class RandomSampleOP : public Operator {
 public:
  explicit RandomSampleOP(int id) : op_id_(id) {}
  void run(OpParams *p) override {
    LMI_MUST(lmi_op_random_sample((lmi_server *)p->env, p->pipe, p->stream, op_id_ / 3 - 1));
  }
 private:
  int op_id_;
};

class CacheLookupOP : public Operator {
 public:
  explicit CacheLookupOP(int id) : op_id_(id) {}
  void run(OpParams *p) override {
    if (p->is_presc) return;  // presampling gathers nothing (engine/operator.cu:73-98)
    LMI_MUST(lmi_op_cache_lookup((lmi_server *)p->env, p->pipe, p->stream, op_id_ / 3));
  }
 private:
  int op_id_;
};

class SSDIOSubmitOP : public Operator {
 public:
  explicit SSDIOSubmitOP(int id) : op_id_(id) {}
  void run(OpParams *p) override { LMI_MUST(lmi_op_io_submit((lmi_server *)p->env, p->pipe, p->stream)); }
 private:
  int op_id_;
};

class SSDIOCompleteOP : public Operator {
 public:
  explicit SSDIOCompleteOP(int id) : op_id_(id) {}
  void run(OpParams *p) override {
    if (p->is_presc) {  // CacheProfiling: count the batch's sampled ids (engine/operator_impl.cu:607-636)
      LMI_MUST(lmi_op_hotness((lmi_server *)p->env, p->pipe, p->stream));
      return;
    }
    LMI_MUST(lmi_op_io_complete((lmi_server *)p->env, p->pipe, p->stream));
  }
 private:
  int op_id_;
};

// ------------------------------------------------------------------- runner
class GPURunner : public Runner {
 public:
  void Initialize(RunnerParams *params) override {
    hops_ = (int)params->fanout.size();
    device_ = params->device_id;
    LMI_MUST(lmi_stream_create(&stream_));
    LMI_MUST(lmi_stream_create(&post_stream_));
    if (IPCEnv *ipc = (IPCEnv *)params->ipc) {  // engine/server.cu:256
      lmi_batch_view v;
      LMI_MUST(lmi_batch_view_get((lmi_server *)params->env, 0, &v));
      ipc->InitializeSamplesBuffer(ipc->GetRawBatchsize(), (int32_t)v.max_nodes, 0, device_, LEGION_INTERBATCH_CON);
    }
    // slot table: [BatchGen, Lookup, IOSubmit, (Sample, Lookup, IOSubmit) x hops, IOComplete]
    ops_.push_back(NewBatchGenerateOP(0));
    ops_.push_back(NewCacheLookupOP(1));
    ops_.push_back(NewSSDIOSubmitOP(2));
    for (int k = 1; k <= hops_; ++k) {
      ops_.push_back(NewRandomSampleOP(3 * k));
      ops_.push_back(NewCacheLookupOP(3 * k + 1));
      ops_.push_back(NewSSDIOSubmitOP(3 * k + 2));
    }
    ops_.push_back(NewSSDIOCompleteOP(3 * (hops_ + 1)));
    op_params_.resize(ops_.size());
    for (size_t i = 0; i < ops_.size(); ++i) {
      OpParams &o = op_params_[i];
      o = OpParams{};
      o.device_id = params->device_id;
      o.stream = stream_;
      o.env = params->env;
      o.in_memory = params->in_memory;
      o.hop_num = hops_;
      o.dyn_cache = params->dyn_cache;
      const int hop = (int)i / 3 - 1;
      o.neighbor_count = (i % 3 == 0 && hop >= 0 && hop < hops_) ? params->fanout[hop] : 0;
    }
  }
  void InitializeFeaturesBuffer(RunnerParams *params) override {  // engine/server.cu:303-308
    if (IPCEnv *ipc = (IPCEnv *)params->ipc) {
      lmi_batch_view v;
      LMI_MUST(lmi_batch_view_get((lmi_server *)params->env, 0, &v));
      ipc->InitializeFeaturesBuffer(0, (int32_t)v.max_nodes, params->feature_dim, device_, LEGION_INTERBATCH_CON);
    }
  }
  void RunPreSc(RunnerParams *params) override { run_table(params, params->global_batch_id, LMI_MODE_TRAIN, true); }
  void RunOnce(RunnerParams *params) override {  // engine/server.cu:330-400
    IPCEnv *ipc = (IPCEnv *)params->ipc;
    int mode = params->mode, local = params->global_batch_id;
    if (ipc) {
      mode = ipc->GetCurrentMode(params->global_batch_id);
      local = ipc->GetLocalBatchId(params->global_batch_id);
    }
    pipe_ ^= 1;  // two output buffer sets, as INTERBATCH_CON = 2
    ran_ = true;
    if (ipc) ipc->IPCWait(device_, pipe_);  // until the trainer has released this buffer set
    if (params->fused) {
      LMI_MUST(lmi_run_once((lmi_server *)params->env, pipe_, stream_, nullptr, 0, LMI_LOC_DEVICE, local, mode, 0));
    } else {
      run_table(params, local, mode, false);
    }
    const bool handoff = ipc && ipc->HandoffEnabled();
    if (handoff) {
      // The batch is posted once it is complete.  With defer_post the one before it is posted now and
      // this one by the next call (or Flush): the device then always has the next batch queued while
      // the host waits for one to finish, and that batch's host-link gather overlaps this one's sampling.
      if (params->defer_post) {
        if (unposted_ >= 0) post(params, unposted_);
        unposted_ = pipe_;
      } else {
        post(params, pipe_);
      }
    } else if (!params->defer_join) {
      LMI_MUST(lmi_batch_wait((lmi_server *)params->env, pipe_, stream_));
    }
  }
  // `count` consecutive batches of the schedule, first = params->global_batch_id, all of one mode,
  // issued together on `count` output buffer sets taken in turn (params->pipes of them exist).
  void RunGroup(RunnerParams *params, int count, int *pipes_out) override {
    IPCEnv *ipc = (IPCEnv *)params->ipc;
    if (count < 1 || count > LMI_MAX_GROUP || count > params->pipes) {
      std::fprintf(stderr, "a group holds 1..%d batches and no more than there are buffer sets\n", LMI_MAX_GROUP);
      std::exit(EXIT_FAILURE);
    }
    int32_t pipes[LMI_MAX_GROUP], counters[LMI_MAX_GROUP];
    int mode = params->mode;
    if (ipc) mode = ipc->GetCurrentMode(params->global_batch_id);
    for (int k = 0; k < count; ++k) {
      pipes[k] = next_pipe_;
      next_pipe_ = (next_pipe_ + 1) % params->pipes;
      counters[k] = ipc ? ipc->GetLocalBatchId(params->global_batch_id + k) : params->global_batch_id + k;
      if (pipes_out) pipes_out[k] = pipes[k];
    }
    pipe_ = pipes[count - 1];
    LMI_MUST(lmi_run_group((lmi_server *)params->env, count, pipes, stream_, nullptr, nullptr, LMI_LOC_DEVICE, counters,
                           mode, nullptr));
  }
  void Flush(RunnerParams *params) override {
    if (unposted_ >= 0) post(params, unposted_);
    unposted_ = -1;
  }
  void Finalize(RunnerParams *params) override {
    Flush(params);
    // the trainer must have released the last batch before its buffers go away
    if (IPCEnv *ipc = (IPCEnv *)params->ipc)
      if (ran_) ipc->IPCWait(device_, pipe_);
    if (stream_) {
      LMI_MUST(lmi_stream_sync(stream_));
      LMI_MUST(lmi_stream_sync(post_stream_));
      LMI_MUST(lmi_stream_destroy(post_stream_));
      LMI_MUST(lmi_stream_destroy(stream_));
      stream_ = post_stream_ = nullptr;
    }
    for (Operator *o : ops_) delete o;
    ops_.clear();
  }
  int CurrentPipe() const override { return pipe_; }
  void *Stream() const override { return stream_; }

 private:
  // Hands the batch in buffer set `pipe` to the trainer once all of it is there.  The wait is for that
  // batch alone -- a stream of its own is put behind the batch's last event and the host waits for that
  // stream -- so a batch queued after it on the runner's stream keeps running meanwhile.
  void post(RunnerParams *params, int pipe) {
    IPCEnv *ipc = (IPCEnv *)params->ipc;
    lmi_server *h = (lmi_server *)params->env;
    LMI_MUST(lmi_batch_wait(h, pipe, post_stream_));
    LMI_MUST(lmi_stream_sync(post_stream_));
    // a batch a kernel flagged (bad seed id, scan that gave up) is never handed over: stop here,
    // as the reference stops on any device error (engine/memorypool.cuh:9-17)
    LMI_MUST(lmi_server_status(h, 0));
    if (ipc->FeaturesInParts(device_)) {  // a feature buffer too large to share whole goes over in pieces
      int32_t nc[16], ec[16];
      LMI_MUST(lmi_batch_counters(h, pipe, post_stream_, nc, ec));
      ipc->StageFeatures(device_, pipe, nc[9 + hops_], post_stream_);
      LMI_MUST(lmi_stream_sync(post_stream_));
    }
    ipc->IPCPost(device_, pipe);
  }
  void run_table(RunnerParams *, int local_batch_id, int mode, bool presc) {
    for (size_t i = 0; i < ops_.size(); ++i) {
      OpParams &o = op_params_[i];
      o.pipe = pipe_;
      o.global_batch_id = local_batch_id;
      o.mode = mode;
      o.is_presc = presc;
      ops_[i]->run(&o);
    }
  }
  int hops_ = 0, pipe_ = 1, device_ = 0;
  int next_pipe_ = 0;   // RunGroup: the buffer set the next batch goes into
  int unposted_ = -1;   // hand-off with defer_post: the buffer set whose batch is issued but not yet posted
  bool ran_ = false;
  void *stream_ = nullptr, *post_stream_ = nullptr;
  std::vector<Operator *> ops_;
  std::vector<OpParams> op_params_;
};

// ------------------------------------------------------------------- server
class GPUServer : public Server {
 public:
  void Initialize(int global_shard_count, std::vector<int> fanout, int in_memory_mode, int dyn_cache) override {
    if (global_shard_count != 1) {
      std::fprintf(stderr, "this build drives one GPU; got gpu_number=%d\n", global_shard_count);
      std::exit(EXIT_FAILURE);
    }
    std::string err;
    const char *meta_path = std::getenv("LEGION_MI_META_CONFIG");
    if (!LegionReadMetaConfig(meta_path ? meta_path : "./meta_config", &meta_, &err)) {
      std::fprintf(stderr, "%s\n", err.c_str());
      std::exit(EXIT_FAILURE);
    }
    fanout_ = fanout;
    dyn_cache_ = dyn_cache;
    lmi_config cfg;
    std::memset(&cfg, 0, sizeof(cfg));
    cfg.device_id = 0;
    cfg.batch_size = meta_.batch_size;
    cfg.hops = (int)fanout.size();
    for (int k = 0; k < cfg.hops && k < LMI_MAX_HOPS; ++k) cfg.fanout[k] = fanout[k];
    cfg.feat_dim = meta_.feature_dim;
    // meta_config has no field for the element type: fp32 as in the reference's files, fp16 on request
    const char *dt = std::getenv("LEGION_MI_FEAT_DTYPE");
    if (dt && std::strcmp(dt, "f16") != 0 && std::strcmp(dt, "f32") != 0) {
      std::fprintf(stderr, "LEGION_MI_FEAT_DTYPE must be f32 or f16, got %s\n", dt);
      std::exit(EXIT_FAILURE);
    }
    elem_bytes_ = (dt && std::strcmp(dt, "f16") == 0) ? 2 : 4;
    cfg.feat_dtype = elem_bytes_ == 2 ? LMI_F16 : LMI_F32;
    cfg.pipes = 2;
    cfg.seed = 1;
    LMI_MUST(lmi_server_create(&cfg, &h_));

    const std::string &dp = meta_.dataset_path;
    const std::string fp = meta_.feature_path.empty() ? dp : meta_.feature_path;
    // topology: int64 row pointers, int32 neighbour ids (dataset/README.md:3-10)
    std::vector<int64_t> indptr((size_t)meta_.node_num + 1);
    std::vector<int32_t> indices((size_t)meta_.edge_num);
    must_read(dp + "edge_src", indptr.data(), (meta_.node_num + 1) * 8);
    must_read(dp + "edge_dst", indices.data(), meta_.edge_num * 4);
    LMI_MUST(lmi_graph_load(h_, indptr.data(), indices.data(), meta_.node_num, meta_.edge_num, LMI_LOC_HOST));
    // features: pinned + mapped host memory, read zero-copy on cache misses
    const int64_t fbytes = meta_.node_num * (int64_t)meta_.feature_dim * elem_bytes_;
    LMI_MUST(lmi_host_alloc((size_t)fbytes, &host_features_));
    must_read(fp + "features", host_features_, fbytes);
    LMI_MUST(lmi_features_attach(h_, host_features_, meta_.node_num, LMI_LOC_HOST));
    // id sets with their labels
    std::vector<int32_t> labels((size_t)meta_.node_num, -1);
    const bool have_labels = read_file(fp + "labels", labels.data(), meta_.node_num * 4) == meta_.node_num * 4;
    const char *names[3] = {"trainingset", "validationset", "testingset"};
    const int64_t counts[3] = {meta_.training_set_num, meta_.validation_set_num, meta_.testing_set_num};
    for (int m = 0; m < 3; ++m) {
      if (counts[m] <= 0) continue;
      std::vector<int32_t> ids((size_t)counts[m]), lab((size_t)counts[m], -1);
      must_read(dp + names[m], ids.data(), counts[m] * 4);
      if (have_labels)
        for (int64_t i = 0; i < counts[m]; ++i)
          if (ids[i] >= 0 && ids[i] < meta_.node_num) lab[i] = labels[ids[i]];
      LMI_MUST(lmi_idset_load(h_, m, ids.data(), have_labels ? lab.data() : nullptr, counts[m], LMI_LOC_HOST));
    }
    // schedule and hand-off (storage_management.cu builds the IPCEnv and calls Coordinate)
    ipc_ = NewIPCEnv(1);
    ipc_->EnableHandoff(handoff_ || std::getenv("LEGION_MI_HANDOFF") != nullptr);
    if (const char *ws = std::getenv("LEGION_MI_WAIT_SECONDS")) wait_seconds_ = std::atof(ws);
    ipc_->SetWaitSeconds(wait_seconds_);
    BuildInfo info;
    info.partition_count = 1;
    info.training_set_num = {(int32_t)meta_.training_set_num};
    info.validation_set_num = {(int32_t)meta_.validation_set_num};
    info.testing_set_num = {(int32_t)meta_.testing_set_num};
    info.epoch = meta_.epoch;
    info.raw_batch_size = meta_.batch_size;
    ipc_->Coordinate(&info);
    for (int m = LMI_MODE_VALID; m <= LMI_MODE_TEST; ++m)
      if (ipc_->GetCurrentBatchsize(0, m) > 0) LMI_MUST(lmi_idset_batch(h_, m, ipc_->GetCurrentBatchsize(0, m)));
    ipc_->BindServer(0, h_);
    runner_ = NewGPURunner();
    params_.ipc = ipc_;
    params_.feature_dim = meta_.feature_dim;
    params_.device_id = 0;
    params_.fanout = fanout;
    params_.cache = params_.graph = params_.feature = nullptr;
    params_.env = h_;
    params_.global_batch_id = 0;
    params_.in_memory = in_memory_mode != 0;
    params_.dyn_cache = dyn_cache;
    params_.fused = std::getenv("LEGION_MI_OPERATOR_TABLE") == nullptr;
    // LEGION_MI_TUNE="key=value,key=value": the library's tuning keys (lmi_tune) for deployments that know
    // their workload, e.g. "split_lookup=2,miss_blocks=48"; none changes a result
    if (const char *tune = std::getenv("LEGION_MI_TUNE")) {
      std::istringstream list(tune);
      std::string item;
      while (std::getline(list, item, ',')) {
        const size_t eq = item.find('=');
        if (item.empty()) continue;
        if (eq == std::string::npos || eq == 0 || eq + 1 >= item.size()) {
          std::fprintf(stderr, "LEGION_MI_TUNE: '%s' is not key=value\n", item.c_str());
          std::exit(EXIT_FAILURE);
        }
        LMI_MUST(lmi_tune(h_, item.substr(0, eq).c_str(), std::atoll(item.c_str() + eq + 1)));
      }
    }
    runner_->Initialize(&params_);
    std::cout << "Storage Initialized\n";
  }

  void PreSc(int cache_agg_mode) override {
    if (cache_agg_mode != 0) {
      std::fprintf(stderr, "cache aggregation across GPUs is not part of this build (mode %d)\n", cache_agg_mode);
      std::exit(EXIT_FAILURE);
    }
    const int64_t row_bytes = (int64_t)meta_.feature_dim * elem_bytes_;
    if (std::getenv("LEGION_MI_PRESAMPLE")) {
      // the reference's policy: one presampling pass over the training set through the
      // operator table, then rank by how often each node was sampled (engine/server.cu:31-37,94-122)
      int32_t steps = 0;
      LMI_MUST(lmi_steps_per_epoch(h_, LMI_MODE_TRAIN, &steps));
      for (int i = 0; i < steps; ++i) {
        params_.global_batch_id = i;
        runner_->RunPreSc(&params_);
      }
      LMI_MUST(lmi_cache_policy(h_, LMI_POLICY_PRESAMPLED));
    }
    runner_->InitializeFeaturesBuffer(&params_);  // engine/server.cu:36
    if (dyn_cache_ & LEGION_DYN_COMP) {
      const int64_t rows = std::max<int64_t>(1, meta_.cache_memory / (meta_.feature_dim + 4));
      LMI_MUST(lmi_cache_build_int8(h_, rows, LMI_TABLE_RANK));
    } else if (dyn_cache_ & LEGION_DYN_ENABLE) {
      const int ways = 8;  // cache/cache.cu:629
      const int64_t sets = std::max<int64_t>(1, meta_.cache_memory / row_bytes / ways);
      LMI_MUST(lmi_cache_build_lru(h_, sets, ways));
    } else {
      const int64_t rows = std::max<int64_t>(1, meta_.cache_memory / row_bytes);
      LMI_MUST(lmi_cache_build_static(h_, rows, LMI_TABLE_RANK));
    }
    lmi_cache_info ci;
    LMI_MUST(lmi_cache_info_get(h_, &ci));
    std::cout << "Cache rows: " << ci.capacity_rows << " (" << ci.capacity_rows * ci.row_bytes << " bytes)\n";
    std::cout << "System is ready for serving" << std::endl;  // the line the reference's scripts wait for
  }

  void Run() override {  // engine/server.cu:124-135
    const int32_t max_step = ipc_->GetMaxStep();
    const bool handoff = ipc_->HandoffEnabled();
    // Batches go out in groups (every launch of a group serves all its batches, lmi_run_group) unless
    // something takes them one by one: the trainer's two buffer sets and their semaphores, the LRU
    // cache (its state advances batch by batch), the operator table.  LEGION_MI_GROUP=1 restores the
    // reference's one batch per RunOnce; LEGION_MI_PIPES sets the number of buffer sets (default: two
    // groups' worth, so that one group's host-link gather overlaps the next group's sampling).
    int group = LMI_MAX_GROUP;
    if (const char *g = std::getenv("LEGION_MI_GROUP")) group = std::max(1, std::min(LMI_MAX_GROUP, std::atoi(g)));
    const bool lru = (dyn_cache_ & LEGION_DYN_ENABLE) && !(dyn_cache_ & LEGION_DYN_COMP);
    if (handoff || lru || !params_.fused) group = 1;
    const auto t0 = std::chrono::steady_clock::now();
    int64_t batches = 0;
    if (group > 1) {
      int pipes = 2 * group;
      if (const char *p = std::getenv("LEGION_MI_PIPES")) pipes = std::max(group, std::min(LMI_MAX_PIPES, std::atoi(p)));
      LMI_MUST(lmi_server_pipes(h_, pipes));
      params_.pipes = pipes;
      batches = run_groups(max_step, group);
    } else {
      // with nobody reading the batches as they come (no sink, no trainer), a batch's host-link
      // gather may run on beside the next batch's sampling; a trainer gets batch i while i + 1 runs
      params_.defer_join = !sink_ && !handoff;
      params_.defer_post = handoff;
      for (int32_t batch_id = 0; batch_id < max_step; ++batch_id) {
        params_.global_batch_id = batch_id;
        runner_->RunOnce(&params_);
        if (sink_) deliver(runner_->CurrentPipe());
        ++batches;
        LMI_MUST(lmi_server_status(h_, 0));  // a host-memory read: conditions of finished batches
      }
      runner_->Flush(&params_);
      for (int pipe = 0; pipe < LEGION_INTERBATCH_CON; ++pipe) LMI_MUST(lmi_batch_wait(h_, pipe, runner_->Stream()));
    }
    LMI_MUST(lmi_stream_sync(runner_->Stream()));
    LMI_MUST(lmi_server_status(h_, 0));  // and those of the last ones
    const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
    std::printf("batches: %lld  time per sample: %.1f us  (%.1f batches/s)\n", (long long)batches,
                batches ? sec * 1e6 / batches : 0.0, sec > 0 ? batches / sec : 0.0);
  }

  void Finalize() override {
    if (runner_) {
      runner_->Finalize(&params_);
      delete runner_;
      runner_ = nullptr;
    }
    if (ipc_) {
      ipc_->Finalize();
      delete ipc_;
      ipc_ = nullptr;
    }
    if (h_) LMI_MUST(lmi_server_destroy(h_));
    h_ = nullptr;
    if (host_features_) LMI_MUST(lmi_host_free(host_features_));
    host_features_ = nullptr;
  }

  void SetBatchSink(LegionBatchSink sink, void *user) override {
    sink_ = sink;
    sink_user_ = user;
  }
  void EnableHandoff(bool on, double wait_seconds) override {
    handoff_ = on;
    wait_seconds_ = wait_seconds;
  }
  lmi_server *Handle(int) override { return h_; }

 private:
  // The sink's turn for the batch in buffer set `pipe`: the stream is put behind all of the batch first.
  void deliver(int pipe) {
    lmi_batch_view v;
    LMI_MUST(lmi_batch_wait(h_, pipe, runner_->Stream()));
    LMI_MUST(lmi_batch_view_get(h_, pipe, &v));
    sink_(&v, 0, pipe, runner_->Stream(), sink_user_);
  }

  // The schedule in groups of at most `group` batches of one mode (a run of r such batches goes out as
  // the fewest groups, sized evenly).  A sink sees the batches of a group, in order, after the NEXT
  // group has been issued: the device keeps working while the host handles them, and the buffer sets
  // of a group are not written again before the group after the next.
  int64_t run_groups(int32_t max_step, int group) {
    std::vector<int> before, now;
    int64_t batches = 0;
    int32_t b = 0;
    while (b < max_step) {
      const int mode = ipc_->GetCurrentMode(b);
      int32_t run = 1;
      while (b + run < max_step && ipc_->GetCurrentMode(b + run) == mode) ++run;
      const int32_t n_groups = (run + group - 1) / group;
      for (int32_t g = 0; g < n_groups; ++g) {
        const int count = run / n_groups + (g < run % n_groups ? 1 : 0);
        now.assign((size_t)count, 0);
        params_.global_batch_id = b;
        runner_->RunGroup(&params_, count, now.data());
        if (sink_)
          for (int pipe : before) deliver(pipe);
        before = now;
        b += count;
        batches += count;
        LMI_MUST(lmi_server_status(h_, 0));  // a host-memory read: conditions of finished batches
      }
    }
    if (sink_)
      for (int pipe : before) deliver(pipe);
    for (int pipe = 0; pipe < params_.pipes; ++pipe) LMI_MUST(lmi_batch_wait(h_, pipe, runner_->Stream()));
    return batches;
  }

  LegionMetaConfig meta_;
  std::vector<int> fanout_;
  int dyn_cache_ = 0;
  int elem_bytes_ = 4;  // of a feature element: fp32, or fp16 with LEGION_MI_FEAT_DTYPE=f16
  lmi_server *h_ = nullptr;
  void *host_features_ = nullptr;
  Runner *runner_ = nullptr;
  IPCEnv *ipc_ = nullptr;
  bool handoff_ = false;
  double wait_seconds_ = 600.0;
  RunnerParams params_{};
  LegionBatchSink sink_ = nullptr;
  void *sink_user_ = nullptr;
};

}  // namespace

bool LegionReadMetaConfig(const std::string &path, LegionMetaConfig *out, std::string *error) {
  std::ifstream f(path);
  if (!f.is_open()) {
    if (error) *error = "unable to open meta config file " + path;
    return false;
  }
  std::string line;
  std::getline(f, line);
  std::istringstream iss(line);
  LegionMetaConfig m;
  if (!(iss >> m.dataset_path >> m.batch_size >> m.node_num >> m.edge_num >> m.feature_dim >> m.training_set_num >>
        m.validation_set_num >> m.testing_set_num >> m.cache_memory >> m.epoch)) {
    if (error) *error = "meta config needs: path batch nodes edges dim train valid test cache_bytes epoch [feat_path]";
    return false;
  }
  iss >> m.feature_path;  // optional
  if (m.batch_size < 1 || m.node_num < 1 || m.edge_num < 0 || m.feature_dim < 1 || m.epoch < 0) {
    if (error) *error = "meta config holds a non-positive size";
    return false;
  }
  if (!m.dataset_path.empty() && m.dataset_path.back() != '/') m.dataset_path += '/';
  if (!m.feature_path.empty() && m.feature_path.back() != '/') m.feature_path += '/';
  *out = m;
  return true;
}

Server *NewGPUServer() { return new GPUServer(); }
Runner *NewGPURunner() { return new GPURunner(); }
Operator *NewBatchGenerateOP(int op_id) { return new BatchGenerateOP(op_id); }
Operator *NewRandomSampleOP(int op_id) { return new RandomSampleOP(op_id); }
Operator *NewCacheLookupOP(int op_id) { return new CacheLookupOP(op_id); }
Operator *NewSSDIOSubmitOP(int op_id) { return new SSDIOSubmitOP(op_id); }
Operator *NewSSDIOCompleteOP(int op_id) { return new SSDIOCompleteOP(op_id); }

// ------------------------------------------------- server on a background thread
namespace {
struct Background {
  std::thread thread;
  std::mutex mu;
  std::condition_variable cv;
  bool ready = false;
  bool started = false;
};
Background g_bg;
}  // namespace

extern "C" int legion_server_start(int gpu_number, int cache_agg_mode, int dyn_cache, const int32_t *fanout,
                                   int hops, int handoff, double wait_seconds) {
  if (g_bg.started || !fanout || hops < 1) return -1;
  std::vector<int> fan(fanout, fanout + hops);
  g_bg.ready = false;
  g_bg.started = true;
  g_bg.thread = std::thread([=]() {
    Server *server = NewGPUServer();
    server->EnableHandoff(handoff != 0, wait_seconds);
    server->Initialize(gpu_number, fan, 1, dyn_cache);
    server->PreSc(cache_agg_mode);
    {
      std::lock_guard<std::mutex> lock(g_bg.mu);
      g_bg.ready = true;
    }
    g_bg.cv.notify_all();
    server->Run();
    server->Finalize();
    delete server;
  });
  std::unique_lock<std::mutex> lock(g_bg.mu);
  g_bg.cv.wait(lock, [] { return g_bg.ready; });
  return 0;
}

extern "C" int legion_server_join(void) {
  if (!g_bg.started) return -1;
  g_bg.thread.join();
  g_bg.started = false;
  return 0;
}
