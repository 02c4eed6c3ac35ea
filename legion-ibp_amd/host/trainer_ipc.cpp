// Trainer-side end of the hand-off (see trainer_ipc.hpp).  Plain C++17 + POSIX; device
// interaction goes through the C ABI: opening the sampler's buffers (lmi_ipc_open), copying
// the two 16-int headers to the host, and putting a feature buffer that arrives in pieces
// together again.
#include "trainer_ipc.hpp"

#include <fcntl.h>
#include <unistd.h>

#include <algorithm>
#include <cerrno>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include "ipc_service.hpp"

namespace legion_trainer {
namespace {

class HostIPCEnv : public IPCEnv {
 public:
  int Initialize() override {
    const int device = 0;  // one GPU
    std::string err;
    shm_ = LegionShmOpen(false, &err);
    if (!shm_) return set_error(err);
    train_step_ = shm_->steps[0];
    valid_step_ = shm_->steps[1];
    test_step_ = shm_->steps[2];
    for (int i = 0; i < LEGION_INTERBATCH_CON; ++i) {
      for (int b = 0; b < LEGION_MEMORY_USAGE; ++b) {
        const LegionBufferHandle &h = shm_->memHandle[device][i][b];
        if (__atomic_load_n(&h.magic, __ATOMIC_ACQUIRE) != LEGION_HANDLE_MAGIC)
          return set_error("buffer set " + std::to_string(i) + " is not exported yet");
        if (b == LEGION_BUF_FEATURES && h.n_parts > 0) {  // handed over in pieces
          if (h.n_parts > LEGION_MAX_FEATURE_PARTS || h.rows_per_part == 0 || h.row_bytes == 0)
            return set_error("the feature buffer's piece table is malformed");
          for (uint32_t k = 0; k < h.n_parts; ++k) {
            const LegionBufferHandle &ph = shm_->featPart[device][i][k];
            if (__atomic_load_n(&ph.magic, __ATOMIC_ACQUIRE) != LEGION_HANDLE_MAGIC)
              return set_error("a piece of the feature buffer is not exported yet");
            void *piece = map_buffer(ph);
            if (!piece) return -1;
            part_[i][k] = piece;
          }
          n_parts_ = (int)h.n_parts;
          rows_per_part_ = (int64_t)h.rows_per_part;
          row_bytes_ = (int64_t)h.row_bytes;
          if (!whole_ && lmi_device_alloc((size_t)h.bytes, &whole_) != LMI_OK) return set_error(lmi_last_error());
          buf_[i][b] = whole_;
          continue;
        }
        buf_[i][b] = map_buffer(h);
        if (!buf_[i][b]) return -1;
      }
      semr_[i] = sem_open(LegionSemName('r', device, i).c_str(), O_RDWR);
      semw_[i] = sem_open(LegionSemName('w', device, i).c_str(), O_RDWR);
      if (semr_[i] == SEM_FAILED || semw_[i] == SEM_FAILED) return set_error(std::string("sem_open: ") + std::strerror(errno));
    }
    // both buffer sets start out free for the sampler
    for (int i = 0; i < LEGION_INTERBATCH_CON; ++i) sem_post(semr_[i]);
    current_pipe_ = 0;
    ready_ = true;
    return device;
  }
  // The rows of a batch whose feature buffer arrives in pieces, put together in a buffer of this
  // process; a no-op otherwise.  After Wait(), before the features are read.
  int Assemble(int64_t n_rows) override {
    if (n_parts_ == 0) return 0;
    for (int k = 0; k < n_parts_; ++k) {
      const int64_t lo = (int64_t)k * rows_per_part_;
      if (lo >= n_rows) break;
      const int64_t rows = std::min<int64_t>(rows_per_part_, n_rows - lo);
      if (lmi_copy_device((char *)whole_ + lo * row_bytes_, part_[current_pipe_][k], (size_t)(rows * row_bytes_), nullptr) != LMI_OK)
        return set_error(lmi_last_error());
    }
    if (lmi_stream_sync(nullptr) != LMI_OK) return set_error(lmi_last_error());
    return 0;
  }
  int32_t *GetIds() override { return (int32_t *)buf_[current_pipe_][LEGION_BUF_IDS]; }
  float *GetFloatFeatures() override { return (float *)buf_[current_pipe_][LEGION_BUF_FEATURES]; }
  int32_t *GetLabels() override { return (int32_t *)buf_[current_pipe_][LEGION_BUF_LABELS]; }
  int32_t *GetAggSrc() override { return (int32_t *)buf_[current_pipe_][LEGION_BUF_AGG_SRC]; }
  int32_t *GetAggDst() override { return (int32_t *)buf_[current_pipe_][LEGION_BUF_AGG_DST]; }
  int32_t *GetNodeCounter() override { return (int32_t *)buf_[current_pipe_][LEGION_BUF_NODE_COUNTER]; }
  int32_t *GetEdgeCounter() override { return (int32_t *)buf_[current_pipe_][LEGION_BUF_EDGE_COUNTER]; }
  int32_t GetTrainStep() override { return train_step_; }
  int32_t GetValidStep() override { return valid_step_; }
  int32_t GetTestStep() override { return test_step_; }
  void Finalize() override {
    for (auto &kv : opened_) lmi_ipc_close(kv.second);  // mappings of another process's allocations
    opened_.clear();
    if (whole_) lmi_device_free(whole_);
    whole_ = nullptr;
    n_parts_ = 0;
    for (int i = 0; i < LEGION_INTERBATCH_CON; ++i) {
      if (semr_[i] && semr_[i] != SEM_FAILED) sem_close(semr_[i]);
      if (semw_[i] && semw_[i] != SEM_FAILED) sem_close(semw_[i]);
      semr_[i] = semw_[i] = nullptr;
    }
    LegionShmClose(shm_);
    shm_ = nullptr;
    ready_ = false;
  }
  void Wait() override { (void)TimedWait(1e9); }
  bool TimedWait(double seconds) override {
    if (!ready_) return false;
    return LegionSemWait(semw_[current_pipe_], seconds);
  }
  void Post() override {
    if (!ready_) return;
    sem_post(semr_[current_pipe_]);
    current_pipe_ = (current_pipe_ + 1) % LEGION_INTERBATCH_CON;
  }
  const char *LastError() const override { return error_.c_str(); }

 private:
  int set_error(const std::string &e) {
    error_ = e;
    return -1;
  }
  // Address of an exported buffer in this process: the exporter's own address when that is this
  // process, otherwise base of the opened allocation (each distinct handle is opened once: the
  // two headers of a buffer set share an allocation) plus the buffer's offset in it.
  void *map_buffer(const LegionBufferHandle &h) {
    if (h.pid == (int64_t)getpid()) return (void *)(uintptr_t)h.address;
    const std::string key((const char *)h.ipc, sizeof(h.ipc));
    auto it = opened_.find(key);
    if (it == opened_.end()) {
      void *base = nullptr;
      if (lmi_ipc_open(h.ipc, &base) != LMI_OK) {
        set_error(std::string("cannot open a buffer of process ") + std::to_string(h.pid) + ": " + lmi_last_error());
        return nullptr;
      }
      it = opened_.emplace(key, base).first;
    }
    return (char *)it->second + h.offset;
  }
  LegionShm *shm_ = nullptr;
  void *buf_[LEGION_INTERBATCH_CON][LEGION_MEMORY_USAGE] = {};
  std::map<std::string, void *> opened_;  // inter-process handle -> base address of its mapping here
  void *part_[LEGION_INTERBATCH_CON][LEGION_MAX_FEATURE_PARTS] = {};
  int n_parts_ = 0;
  int64_t rows_per_part_ = 0, row_bytes_ = 0;
  void *whole_ = nullptr;  // this process's own buffer for a feature buffer that arrives in pieces
  sem_t *semr_[LEGION_INTERBATCH_CON] = {}, *semw_[LEGION_INTERBATCH_CON] = {};
  int32_t train_step_ = 0, valid_step_ = 0, test_step_ = 0;
  int current_pipe_ = 0;
  bool ready_ = false;
  std::string error_;
};

}  // namespace

IPCEnv *NewIPCEnv() { return new HostIPCEnv(); }

}  // namespace legion_trainer

// ------------------------------------------------------------------ C interface
namespace {
legion_trainer::IPCEnv *g_env = nullptr;
int32_t g_node_counter[16], g_edge_counter[16];
std::string g_error;
}  // namespace

extern "C" int legion_ipc_initialize(void) {
  if (g_env) {
    g_env->Finalize();
    delete g_env;
  }
  g_env = legion_trainer::NewIPCEnv();
  std::memset(g_node_counter, 0, sizeof(g_node_counter));
  std::memset(g_edge_counter, 0, sizeof(g_edge_counter));
  if (g_env->Initialize() < 0) {
    g_error = g_env->LastError();
    g_env->Finalize();  // whatever it had opened before it failed
    delete g_env;
    g_env = nullptr;
    return -1;
  }
  return 0;
}

extern "C" const char *legion_ipc_last_error(void) { return g_error.c_str(); }

extern "C" int legion_ipc_get_next(legion_ipc_batch *out, double wait_seconds) {
  if (!g_env || !out) {
    g_error = "legion_ipc_initialize has not succeeded";
    return -1;
  }
  if (!g_env->TimedWait(wait_seconds)) {
    g_error = "no batch arrived in time";
    return -1;
  }
  if (lmi_copy_to_host(g_node_counter, g_env->GetNodeCounter(), 64) != LMI_OK ||
      lmi_copy_to_host(g_edge_counter, g_env->GetEdgeCounter(), 64) != LMI_OK) {
    g_error = lmi_last_error();
    return -1;
  }
  std::memset(out, 0, sizeof(*out));
  std::memcpy(out->node_counter, g_node_counter, 64);
  std::memcpy(out->edge_counter, g_edge_counter, 64);
  const int hops = g_node_counter[8];
  if (hops < 0 || hops > LEGION_IPC_MAX_HOPS) {
    g_error = "the batch header names " + std::to_string(hops) + " hops";
    return -1;
  }
  out->hop_num = hops;
  out->ids = g_env->GetIds();
  out->n_ids = g_node_counter[9 + hops];
  if (g_env->Assemble(out->n_ids) != 0) {
    g_error = g_env->LastError();
    return -1;
  }
  out->features = g_env->GetFloatFeatures();
  out->labels = g_env->GetLabels();
  out->n_labels = g_node_counter[9];
  for (int i = hops, k = 0; i > 0; --i, ++k) {
    out->agg_src[k] = g_env->GetAggSrc() + g_edge_counter[12 + i];
    out->agg_dst[k] = g_env->GetAggDst() + g_edge_counter[12 + i];
    out->n_edges[k] = g_edge_counter[9 + i];
  }
  return 0;
}

extern "C" int legion_ipc_get_block_size(int32_t *out, int capacity) {
  const int hops = g_node_counter[8];
  int n = 0;
  for (int i = hops; i > 0 && n + 2 <= capacity; --i) {
    out[n++] = g_node_counter[9 + i];
    out[n++] = g_node_counter[9 + i - 1];
  }
  return n;
}

extern "C" void legion_ipc_get_steps(int32_t steps[3]) {
  steps[0] = g_env ? g_env->GetTrainStep() : 0;
  steps[1] = g_env ? g_env->GetValidStep() : 0;
  steps[2] = g_env ? g_env->GetTestStep() : 0;
}

extern "C" void legion_ipc_synchronize(void) {
  if (g_env) g_env->Post();
}

extern "C" void legion_ipc_finalize(void) {
  if (!g_env) return;
  g_env->Finalize();
  delete g_env;
  g_env = nullptr;
}
