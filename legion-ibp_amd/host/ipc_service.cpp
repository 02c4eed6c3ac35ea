// Sampler-side hand-off environment (see ipc_service.hpp).  Plain C++17 + POSIX.
//
// Reference behaviour followed here (Legion-IBP sampling_server/src/engine):
//   ipc_service.cu:60-128    Coordinate: step counts and per-mode batch sizes
//   ipc_service.cu:130-206   buffer export + semaphores per (device, buffer set)
//   ipc_service.cu:212-260   global batch id -> (mode, local batch id)
//   ipc_service.cu:283-291   IPCPost / IPCWait
//   helper_multiprocess.cu:32-69   the shared-memory slab
#include "ipc_service.hpp"

#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <time.h>
#include <unistd.h>

#include <algorithm>
#include <array>
#include <cerrno>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <iostream>

LegionShm *LegionShmOpen(bool create, std::string *error) {
  const int fd = shm_open(LEGION_SHM_NAME, create ? (O_RDWR | O_CREAT) : O_RDWR, 0666);
  if (fd < 0) {
    if (error) *error = std::string("shm_open(" LEGION_SHM_NAME "): ") + std::strerror(errno);
    return nullptr;
  }
  if (create && ftruncate(fd, (off_t)sizeof(LegionShm)) != 0) {
    if (error) *error = std::string("ftruncate(" LEGION_SHM_NAME "): ") + std::strerror(errno);
    close(fd);
    return nullptr;
  }
  struct stat sb;
  if (fstat(fd, &sb) != 0 || (size_t)sb.st_size < sizeof(LegionShm)) {
    if (error) *error = LEGION_SHM_NAME " is smaller than the hand-off slab: no sampling server has set it up";
    close(fd);
    return nullptr;
  }
  void *addr = mmap(nullptr, sizeof(LegionShm), PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0);
  close(fd);
  if (addr == MAP_FAILED) {
    if (error) *error = std::string("mmap(" LEGION_SHM_NAME "): ") + std::strerror(errno);
    return nullptr;
  }
  return (LegionShm *)addr;
}

void LegionShmClose(LegionShm *shm) {
  if (shm) munmap((void *)shm, sizeof(LegionShm));
}

std::string LegionSemName(char kind, int device, int set) {
  return std::string("/sem_") + kind + "_" + std::to_string(device) + "_" + std::to_string(set);
}

bool LegionSemWait(sem_t *sem, double seconds) {
  struct timespec ts;
  clock_gettime(CLOCK_REALTIME, &ts);
  const double whole = (double)(int64_t)seconds;
  ts.tv_sec += (time_t)whole;
  ts.tv_nsec += (long)((seconds - whole) * 1e9);
  if (ts.tv_nsec >= 1000000000L) {
    ts.tv_sec += 1;
    ts.tv_nsec -= 1000000000L;
  }
  while (true) {
    if (sem_timedwait(sem, &ts) == 0) return true;
    if (errno == EINTR) continue;
    return false;
  }
}

namespace {

[[noreturn]] void fail(const std::string &what) {
  std::fprintf(stderr, "legion hand-off: %s\n", what.c_str());
  std::exit(EXIT_FAILURE);
}

class HostIPCEnv : public IPCEnv {
 public:
  explicit HostIPCEnv(int32_t device_count) : device_count_(device_count) {
    if (device_count < 1 || device_count > LEGION_MAX_DEVICE) fail("device count outside 1.." + std::to_string(LEGION_MAX_DEVICE));
    servers_.assign((size_t)device_count, nullptr);
    views_.assign((size_t)device_count, std::vector<lmi_batch_view>());
    semr_.assign((size_t)device_count, std::vector<sem_t *>());
    semw_.assign((size_t)device_count, std::vector<sem_t *>());
    parts_.resize((size_t)device_count);
  }

  void EnableHandoff(bool on) override { handoff_ = on; }
  bool HandoffEnabled() const override { return handoff_; }
  void SetWaitSeconds(double seconds) override { wait_seconds_ = seconds; }
  void BindServer(int32_t device_id, lmi_server *server) override { servers_.at((size_t)device_id) = server; }

  void Coordinate(BuildInfo *info) override {
    const int32_t parts = info->partition_count;
    epoch_ = info->epoch;
    raw_batch_size_ = info->raw_batch_size;
    if (raw_batch_size_ < 1) fail("raw batch size must be positive");
    // training: every partition runs the step count of the smallest one; the last,
    // possibly short, batch of the set is not served
    int32_t min_train = 1000000000;
    for (int32_t i = 0; i < parts; ++i) min_train = std::min(min_train, info->training_set_num[(size_t)i]);
    train_step_ = min_train > 0 ? (min_train - 1) / raw_batch_size_ : 0;
    train_batch_size_.assign((size_t)parts, raw_batch_size_);
    // validation and test: steps from the largest partition at 512 ids a step (no more than
    // the output buffers hold), then every partition spreads its ids evenly over those steps
    const int32_t raw_eval = std::min<int32_t>(LEGION_VALID_TEST_RAW_BATCH, raw_batch_size_);
    spread(info->validation_set_num, parts, raw_eval, &valid_step_, &valid_batch_size_);
    spread(info->testing_set_num, parts, raw_eval, &test_step_, &test_batch_size_);
    std::cout << "Train Steps: " << train_step_ << "\n";
    std::cout << "Valid Steps: " << valid_step_ << "\n";
    std::cout << "Test Steps: " << test_step_ << "\n";
    if (handoff_) {
      std::string err;
      shm_ = LegionShmOpen(true, &err);
      if (!shm_) fail(err);
      std::memset((void *)shm_, 0, sizeof(*shm_));
      shm_->steps[0] = train_step_;
      shm_->steps[1] = valid_step_;
      shm_->steps[2] = test_step_;
    }
  }

  int32_t GetMaxStep() override { return (train_step_ + valid_step_) * epoch_ + test_step_; }

  void InitializeSamplesBuffer(int32_t batch_size, int32_t num_ids, int32_t feature_dim, int32_t device_id,
                               int32_t pipeline_depth) override {
    (void)feature_dim;
    lmi_server *srv = servers_.at((size_t)device_id);
    if (!srv) fail("BindServer must come before InitializeSamplesBuffer");
    if (pipeline_depth < 1 || pipeline_depth > LEGION_INTERBATCH_CON) fail("pipeline depth outside 1..2");
    pipeline_depth_ = pipeline_depth;
    auto &views = views_[(size_t)device_id];
    views.resize((size_t)pipeline_depth);
    for (int32_t i = 0; i < pipeline_depth; ++i) {
      if (lmi_batch_view_get(srv, i, &views[(size_t)i]) != LMI_OK) fail(std::string("lmi_batch_view_get: ") + lmi_last_error());
      if (views[(size_t)i].max_nodes < num_ids) fail("the server's output buffers hold fewer ids than asked for");
    }
    if (!handoff_) return;
    semr_[(size_t)device_id].resize((size_t)pipeline_depth);
    semw_[(size_t)device_id].resize((size_t)pipeline_depth);
    for (int32_t i = 0; i < pipeline_depth; ++i) {
      const lmi_batch_view &v = views[(size_t)i];
      publish(device_id, i, LEGION_BUF_IDS, v.ids, (uint64_t)v.max_nodes * 4);
      publish(device_id, i, LEGION_BUF_LABELS, v.labels, (uint64_t)batch_size * 4);
      publish(device_id, i, LEGION_BUF_AGG_SRC, v.agg_src_off, (uint64_t)v.max_edges * 4);
      publish(device_id, i, LEGION_BUF_AGG_DST, v.agg_dst_off, (uint64_t)v.max_edges * 4);
      publish(device_id, i, LEGION_BUF_NODE_COUNTER, v.node_counter, 64);
      publish(device_id, i, LEGION_BUF_EDGE_COUNTER, v.edge_counter, 64);
      // semaphores start at 0; one left behind by a run that died is removed first
      const std::string nr = LegionSemName('r', device_id, i), nw = LegionSemName('w', device_id, i);
      sem_unlink(nr.c_str());
      sem_unlink(nw.c_str());
      semr_[(size_t)device_id][(size_t)i] = sem_open(nr.c_str(), O_CREAT | O_RDWR, 0666, 0);
      semw_[(size_t)device_id][(size_t)i] = sem_open(nw.c_str(), O_CREAT | O_RDWR, 0666, 0);
      if (semr_[(size_t)device_id][(size_t)i] == SEM_FAILED || semw_[(size_t)device_id][(size_t)i] == SEM_FAILED)
        fail(std::string("sem_open: ") + std::strerror(errno));
    }
  }

  void InitializeFeaturesBuffer(int32_t batch_size, int32_t num_ids, int32_t feature_dim, int32_t device_id,
                                int32_t pipeline_depth) override {
    (void)batch_size;
    (void)num_ids;
    (void)feature_dim;  // the server knows the size of its rows (fp32 or fp16)
    if (!handoff_) return;
    const auto &views = views_.at((size_t)device_id);
    // largest allocation another process can open; smaller on request, to rehearse the split on a small buffer
    uint64_t part_limit = (uint64_t)LMI_IPC_MAX_BYTES - (1u << 24);
    if (const char *e = std::getenv("LEGION_MI_IPC_PART_BYTES")) part_limit = std::strtoull(e, nullptr, 10);
    for (int32_t i = 0; i < pipeline_depth && i < (int32_t)views.size(); ++i) {
      const lmi_batch_view &v = views[(size_t)i];
      const uint64_t row_bytes = (uint64_t)v.row_bytes, total = (uint64_t)v.max_nodes * row_bytes;
      if (total <= part_limit) {
        publish(device_id, i, LEGION_BUF_FEATURES, v.features, total);
        continue;
      }
      // too large to share as one allocation: pieces of their own, filled by StageFeatures
      const uint64_t rows_per_part = part_limit / row_bytes;
      if (rows_per_part < 1) fail("LEGION_MI_IPC_PART_BYTES is smaller than one feature row");
      const uint64_t n_parts = ((uint64_t)v.max_nodes + rows_per_part - 1) / rows_per_part;
      if (n_parts > LEGION_MAX_FEATURE_PARTS)
        fail("a feature buffer of " + std::to_string(total) + " bytes needs more than " +
             std::to_string(LEGION_MAX_FEATURE_PARTS) + " shared pieces");
      LegionBufferHandle &h = shm_->memHandle[device_id][i][LEGION_BUF_FEATURES];
      std::memset(&h, 0, sizeof(h));
      h.pid = (int64_t)getpid();
      h.address = (uint64_t)(uintptr_t)v.features;
      h.bytes = total;
      h.n_parts = (uint32_t)n_parts;
      h.rows_per_part = rows_per_part;
      h.row_bytes = row_bytes;
      for (uint64_t k = 0; k < n_parts; ++k) {
        const uint64_t rows = std::min<uint64_t>(rows_per_part, (uint64_t)v.max_nodes - k * rows_per_part);
        void *piece = nullptr;
        if (lmi_device_alloc((size_t)(rows * row_bytes), &piece) != LMI_OK) fail(std::string("lmi_device_alloc: ") + lmi_last_error());
        parts_[(size_t)device_id][(size_t)i].push_back(piece);
        export_to(&shm_->featPart[device_id][i][k], piece, rows * row_bytes);
      }
      __atomic_store_n(&h.magic, LEGION_HANDLE_MAGIC, __ATOMIC_RELEASE);
    }
  }

  bool FeaturesInParts(int32_t dev_id) const override {
    return handoff_ && !parts_.at((size_t)dev_id)[0].empty();
  }

  void StageFeatures(int32_t dev_id, int32_t current_pipe, int64_t n_rows, void *stream) override {
    if (!handoff_) return;
    const int set = current_pipe % pipeline_depth_;
    const auto &pieces = parts_.at((size_t)dev_id)[(size_t)set];
    if (pieces.empty()) return;
    const LegionBufferHandle &h = shm_->memHandle[dev_id][set][LEGION_BUF_FEATURES];
    const char *src = (const char *)view(dev_id, set).features;
    for (size_t k = 0; k < pieces.size(); ++k) {
      const int64_t lo = (int64_t)(k * h.rows_per_part);
      if (lo >= n_rows) break;
      const int64_t rows = std::min<int64_t>((int64_t)h.rows_per_part, n_rows - lo);
      if (lmi_copy_device(pieces[k], src + lo * (int64_t)h.row_bytes, (size_t)(rows * (int64_t)h.row_bytes), stream) != LMI_OK)
        fail(std::string("lmi_copy_device: ") + lmi_last_error());
    }
  }

  int32_t GetRawBatchsize() override { return raw_batch_size_; }

  int32_t GetLocalBatchId(int32_t global_batch_id) override {
    const int32_t per_epoch = train_step_ + valid_step_;
    if (global_batch_id < per_epoch * epoch_) {
      const int32_t in_epoch = global_batch_id % per_epoch;
      return in_epoch < train_step_ ? in_epoch : in_epoch - train_step_;
    }
    return test_step_ ? (global_batch_id - per_epoch * epoch_) % test_step_ : -1;
  }

  int32_t GetCurrentBatchsize(int32_t dev_id, int32_t current_mode) override {
    if (current_mode == LMI_MODE_TRAIN) return train_batch_size_.at((size_t)dev_id);
    if (current_mode == LMI_MODE_VALID) return valid_batch_size_.at((size_t)dev_id);
    return test_batch_size_.at((size_t)dev_id);
  }

  int32_t GetCurrentMode(int32_t global_batch_id) override {
    const int32_t per_epoch = train_step_ + valid_step_;
    if (global_batch_id < per_epoch * epoch_)
      return (global_batch_id % per_epoch) < train_step_ ? LMI_MODE_TRAIN : LMI_MODE_VALID;
    return LMI_MODE_TEST;
  }

  int32_t *GetIds(int32_t d, int32_t p) override { return view(d, p).ids; }
  float *GetFloatFeatures(int32_t d, int32_t p) override { return (float *)view(d, p).features; }
  int32_t *GetLabels(int32_t d, int32_t p) override { return view(d, p).labels; }
  int32_t *GetAggSrc(int32_t d, int32_t p) override { return view(d, p).agg_src_off; }
  int32_t *GetAggDst(int32_t d, int32_t p) override { return view(d, p).agg_dst_off; }
  int32_t *GetNodeCounter(int32_t d, int32_t p) override { return view(d, p).node_counter; }
  int32_t *GetEdgeCounter(int32_t d, int32_t p) override { return view(d, p).edge_counter; }

  void IPCPost(int32_t dev_id, int32_t current_pipe) override {
    if (!handoff_) return;
    sem_post(semw_.at((size_t)dev_id).at((size_t)(current_pipe % pipeline_depth_)));
  }

  void IPCWait(int32_t dev_id, int32_t current_pipe) override {
    if (!handoff_) return;
    if (!LegionSemWait(semr_.at((size_t)dev_id).at((size_t)(current_pipe % pipeline_depth_)), wait_seconds_))
      fail("no trainer released buffer set " + std::to_string(current_pipe % pipeline_depth_) + " within " +
           std::to_string((int)wait_seconds_) + " s");
  }

  void Finalize() override {
    for (int32_t d = 0; d < device_count_; ++d) {
      for (size_t i = 0; i < semr_[(size_t)d].size(); ++i) {
        if (semr_[(size_t)d][i] && semr_[(size_t)d][i] != SEM_FAILED) sem_close(semr_[(size_t)d][i]);
        if (semw_[(size_t)d][i] && semw_[(size_t)d][i] != SEM_FAILED) sem_close(semw_[(size_t)d][i]);
        sem_unlink(LegionSemName('r', d, (int)i).c_str());
        sem_unlink(LegionSemName('w', d, (int)i).c_str());
      }
      semr_[(size_t)d].clear();
      semw_[(size_t)d].clear();
    }
    for (auto &dev : parts_)
      for (auto &set : dev) {
        for (void *piece : set) lmi_device_free(piece);
        set.clear();
      }
    if (shm_) {
      LegionShmClose(shm_);
      shm_unlink(LEGION_SHM_NAME);
      shm_ = nullptr;
    }
  }

  int32_t GetTrainStep() override { return train_step_; }
  int32_t GetValidStep() override { return valid_step_; }
  int32_t GetTestStep() override { return test_step_; }

 private:
  static void spread(const std::vector<int32_t> &nums, int32_t parts, int32_t raw, int32_t *steps,
                     std::vector<int32_t> *sizes) {
    int32_t largest = 0;
    for (int32_t i = 0; i < parts; ++i) largest = std::max(largest, nums[(size_t)i]);
    *steps = largest > 0 ? (largest - 1) / raw + 1 : 0;
    sizes->assign((size_t)parts, 0);
    for (int32_t i = 0; i < parts; ++i)
      if (*steps && nums[(size_t)i] > 0) (*sizes)[(size_t)i] = (nums[(size_t)i] - 1) / *steps + 1;
  }

  const lmi_batch_view &view(int32_t d, int32_t p) {
    return views_.at((size_t)d).at((size_t)(p % pipeline_depth_));
  }

  void publish(int32_t d, int32_t set, int which, const void *ptr, uint64_t bytes) {
    export_to(&shm_->memHandle[d][set][which], ptr, bytes);
  }

  // Fills a slot with the buffer's inter-process handle (of the allocation that holds it), where
  // the buffer lies in that allocation, and -- for a consumer inside this process -- its address.
  void export_to(LegionBufferHandle *slot, const void *ptr, uint64_t bytes) {
    LegionBufferHandle h;
    std::memset(&h, 0, sizeof(h));
    h.pid = (int64_t)getpid();
    h.address = (uint64_t)(uintptr_t)ptr;
    h.bytes = bytes;
    int64_t offset = 0, alloc_bytes = 0;
    if (lmi_ipc_export(ptr, h.ipc, &offset, &alloc_bytes) != LMI_OK) fail(std::string("lmi_ipc_export: ") + lmi_last_error());
    h.offset = (uint64_t)offset;
    *slot = h;
    __atomic_store_n(&slot->magic, LEGION_HANDLE_MAGIC, __ATOMIC_RELEASE);  // last: the slot is complete
  }

  int32_t device_count_;
  bool handoff_ = false;
  double wait_seconds_ = 600.0;
  LegionShm *shm_ = nullptr;
  std::vector<lmi_server *> servers_;
  std::vector<std::vector<lmi_batch_view>> views_;
  std::vector<std::vector<sem_t *>> semr_, semw_;
  // [device][buffer set]: separately allocated pieces of a feature buffer too large to share whole
  std::vector<std::array<std::vector<void *>, LEGION_INTERBATCH_CON>> parts_;
  int32_t raw_batch_size_ = 0;
  std::vector<int32_t> train_batch_size_, valid_batch_size_, test_batch_size_;
  int32_t train_step_ = 0, valid_step_ = 0, test_step_ = 0;
  int32_t epoch_ = 1;
  int32_t pipeline_depth_ = LEGION_INTERBATCH_CON;
};

}  // namespace

IPCEnv *NewIPCEnv(int32_t device_count) { return new HostIPCEnv(device_count); }

// Schedule of one partition without any server: steps[3] = train, valid, test step counts,
// sizes[3] = ids per batch of each mode.  For host languages that drive the C ABI themselves.
extern "C" void legion_schedule(int32_t train_n, int32_t valid_n, int32_t test_n, int32_t raw_batch, int32_t epoch,
                                int32_t steps[3], int32_t sizes[3], int32_t *max_step) {
  HostIPCEnv env(1);
  BuildInfo info;
  info.training_set_num = {train_n};
  info.validation_set_num = {valid_n};
  info.testing_set_num = {test_n};
  info.epoch = epoch;
  info.raw_batch_size = raw_batch;
  std::cout.setstate(std::ios_base::failbit);  // Coordinate prints the step counts
  env.Coordinate(&info);
  std::cout.clear();
  steps[0] = env.GetTrainStep();
  steps[1] = env.GetValidStep();
  steps[2] = env.GetTestStep();
  for (int m = 0; m < 3; ++m) sizes[m] = env.GetCurrentBatchsize(0, m);
  if (max_step) *max_step = env.GetMaxStep();
}

// (mode, local batch id) of a global batch id under the same schedule.
extern "C" void legion_schedule_batch(int32_t train_n, int32_t valid_n, int32_t test_n, int32_t raw_batch,
                                      int32_t epoch, int32_t global_batch_id, int32_t *mode, int32_t *local_id) {
  HostIPCEnv env(1);
  BuildInfo info;
  info.training_set_num = {train_n};
  info.validation_set_num = {valid_n};
  info.testing_set_num = {test_n};
  info.epoch = epoch;
  info.raw_batch_size = raw_batch;
  std::cout.setstate(std::ios_base::failbit);
  env.Coordinate(&info);
  std::cout.clear();
  *mode = env.GetCurrentMode(global_batch_id);
  *local_id = env.GetLocalBatchId(global_batch_id);
}
