// Sampler-side hand-off to a trainer: batch schedule, exported output buffers and the
// two-semaphore handshake per output buffer set.
//
// Same interface as the reference's IPCEnv (Legion-IBP
// sampling_server/src/engine/ipc_service.h:6-36, implementation
// engine/ipc_service.cu:33-351): the schedule arithmetic (Coordinate, GetMaxStep,
// GetLocalBatchId, GetCurrentMode, GetCurrentBatchsize), the shared-memory slab
// "simpleIPCshm" holding the three step counts and one 64-byte handle per
// (device, buffer set, buffer), and the named semaphores sem_r_<dev>_<set> /
// sem_w_<dev>_<set>.
//
// What differs: the output buffers belong to the lmi_server's pipes (BindServer).  A handle
// slot carries the 64-byte inter-process memory handle of the buffer's allocation
// (lmi_ipc_export; the reference stores a cudaIpcMemHandle_t, engine/ipc_service.cu:163-192)
// plus the exporting process id, the device address there, the buffer's offset inside the
// allocation and its size: a trainer in another process opens the handle, one in the same
// process (another thread) uses the address.  An allocation shared between processes must
// stay under 2 GiB here, so a feature buffer of that size or more is handed over in pieces:
// the sampler copies a finished batch's rows into up to LEGION_MAX_FEATURE_PARTS separately
// allocated pieces (StageFeatures) and the trainer puts them together again.  An empty
// validation or test set has 0 steps (the reference computes 1 step of 0 ids).
#pragma once

#include <semaphore.h>

#include <cstdint>
#include <string>
#include <vector>

#include "../../include/legion_mi.h"

#define LEGION_MAX_DEVICE 8     // MAX_DEVICE     (engine/ipc_service.cu:20)
#define LEGION_INTERBATCH_CON 2 // INTERBATCH_CON (engine/ipc_service.h, memorypool.cuh)
#define LEGION_MEMORY_USAGE 7   // MEMORY_USAGE   (engine/ipc_service.cu:21)
#define LEGION_SHM_NAME "simpleIPCshm"
#define LEGION_VALID_TEST_RAW_BATCH 512  // raw_valid_batch_size / raw_test_batch_size (ipc_service.cu:88,101)

enum LegionBufferIndex {  // order of the handles of one buffer set (engine/ipc_service.cu:164-170)
  LEGION_BUF_IDS = 0, LEGION_BUF_FEATURES = 1, LEGION_BUF_LABELS = 2, LEGION_BUF_AGG_SRC = 3,
  LEGION_BUF_AGG_DST = 4, LEGION_BUF_NODE_COUNTER = 5, LEGION_BUF_EDGE_COUNTER = 6
};

#define LEGION_MAX_FEATURE_PARTS 8  // pieces a feature buffer too large for one shared allocation is handed over in

struct LegionBufferHandle {  // 128 bytes
  uint64_t magic;            // LEGION_HANDLE_MAGIC once exported
  int64_t pid;               // exporting process
  uint64_t address;          // device address of the buffer, valid in that process
  uint64_t bytes;            // size of the buffer
  uint64_t offset;           // of the buffer inside the allocation the handle names
  uint32_t n_parts;          // features only: > 0 = the rows arrive in that many pieces (featPart), not here
  uint32_t reserved;
  uint64_t rows_per_part;    // rows every piece but the last holds
  uint64_t row_bytes;        // features only
  uint8_t ipc[64];           // inter-process memory handle of the allocation (LMI_IPC_HANDLE_BYTES)
};
#define LEGION_HANDLE_MAGIC 0x4c4d49424e444c46ull

struct LegionShm {  // shmStruct (engine/ipc_service.cu:28-31)
  int32_t steps[3];
  int32_t pad;
  LegionBufferHandle memHandle[LEGION_MAX_DEVICE][LEGION_INTERBATCH_CON][LEGION_MEMORY_USAGE];
  LegionBufferHandle featPart[LEGION_MAX_DEVICE][LEGION_INTERBATCH_CON][LEGION_MAX_FEATURE_PARTS];
};

// The fields of the reference's BuildInfo the hand-off reads (include/buildinfo.h:6-80).
struct BuildInfo {
  int32_t partition_count = 1;
  std::vector<int32_t> training_set_num, validation_set_num, testing_set_num;
  int32_t epoch = 1;
  int32_t raw_batch_size = 0;
};

class IPCEnv {
 public:
  virtual ~IPCEnv() {}
  virtual void Coordinate(BuildInfo *info) = 0;
  virtual int32_t GetMaxStep() = 0;

  virtual void InitializeSamplesBuffer(int32_t batch_size, int32_t num_ids, int32_t feature_dim, int32_t device_id,
                                       int32_t pipeline_depth) = 0;
  virtual void InitializeFeaturesBuffer(int32_t batch_size, int32_t num_ids, int32_t feature_dim, int32_t device_id,
                                        int32_t pipeline_depth) = 0;

  virtual int32_t GetRawBatchsize() = 0;
  virtual int32_t GetLocalBatchId(int32_t global_batch_id) = 0;
  virtual int32_t GetCurrentBatchsize(int32_t dev_id, int32_t current_mode) = 0;
  virtual int32_t GetCurrentMode(int32_t global_batch_id) = 0;

  virtual int32_t *GetIds(int32_t dev_id, int32_t current_pipe) = 0;
  virtual float *GetFloatFeatures(int32_t dev_id, int32_t current_pipe) = 0;
  virtual int32_t *GetLabels(int32_t dev_id, int32_t current_pipe) = 0;
  virtual int32_t *GetAggSrc(int32_t dev_id, int32_t current_pipe) = 0;
  virtual int32_t *GetAggDst(int32_t dev_id, int32_t current_pipe) = 0;
  virtual int32_t *GetNodeCounter(int32_t dev_id, int32_t current_pipe) = 0;
  virtual int32_t *GetEdgeCounter(int32_t dev_id, int32_t current_pipe) = 0;

  virtual void IPCPost(int32_t dev_id, int32_t current_pipe) = 0;
  virtual void IPCWait(int32_t dev_id, int32_t current_pipe) = 0;

  virtual void Finalize() = 0;
  virtual int32_t GetTrainStep() = 0;

  // additions
  virtual int32_t GetValidStep() = 0;
  virtual int32_t GetTestStep() = 0;
  // The server whose pipes are the output buffer sets of `device_id`; call before
  // InitializeSamplesBuffer.
  virtual void BindServer(int32_t device_id, lmi_server *server) = 0;
  // Off (default): no shared memory, no semaphores, IPCWait / IPCPost return at once and
  // the sampler free-runs.  On: the handshake of the reference.  Call before Coordinate.
  virtual void EnableHandoff(bool on) = 0;
  virtual bool HandoffEnabled() const = 0;
  // Longest IPCWait before the process gives up (the reference waits for ever).
  virtual void SetWaitSeconds(double seconds) = 0;
  // When the feature buffer of the buffer set is handed over in pieces: copies the first n_rows
  // rows of the set's feature buffer into them, asynchronously on `stream`; otherwise does nothing.
  // Between the end of the batch and IPCPost.
  virtual void StageFeatures(int32_t dev_id, int32_t current_pipe, int64_t n_rows, void *stream) = 0;
  virtual bool FeaturesInParts(int32_t dev_id) const = 0;
};

IPCEnv *NewIPCEnv(int32_t device_count);

// Maps (creating it if need be) the named slab; returns nullptr and fills `error` on failure.
LegionShm *LegionShmOpen(bool create, std::string *error);
void LegionShmClose(LegionShm *shm);
std::string LegionSemName(char kind /* 'r' or 'w' */, int device, int set);
// sem_wait with a deadline; false when the deadline passed.
bool LegionSemWait(sem_t *sem, double seconds);
