// Trainer-side end of the hand-off: opens the output buffer sets a sampling server
// exported and takes one finished mini-batch at a time.
//
// Same interface as the reference's trainer-side IPCEnv and the functions of its
// `ipc_service` extension module (Legion-IBP training_backend/ipc_service.h:6-22,
// ipc_cuda_kernel.cu:35-173 for the class, ipc_service.cpp:15-97 and
// ipc_cuda_kernel.cu:177-240 for initialize / get_next / get_block_size / get_steps /
// synchronize / finalize).  The class lives in a namespace because the sampler-side
// class of the same name may be linked into the same process.
//
// The sampling server may run in another process (the reference's deployment: its buffers are
// opened through the inter-process memory handles of the slab, before this process does any
// other GPU work) or on another thread of this one (the slab's device addresses are used).
#pragma once

#include <cstdint>

#ifdef __cplusplus
namespace legion_trainer {

class IPCEnv {
 public:
  virtual ~IPCEnv() {}
  virtual int Initialize() = 0;  // returns the device (0), or -1 with the reason in LastError()
  virtual int32_t *GetIds() = 0;
  virtual float *GetFloatFeatures() = 0;
  virtual int32_t *GetLabels() = 0;
  virtual int32_t *GetAggSrc() = 0;
  virtual int32_t *GetAggDst() = 0;
  virtual int32_t *GetNodeCounter() = 0;
  virtual int32_t *GetEdgeCounter() = 0;
  virtual int32_t GetTrainStep() = 0;
  virtual int32_t GetValidStep() = 0;
  virtual int32_t GetTestStep() = 0;
  virtual void Finalize() = 0;
  virtual void Wait() = 0;  // until the sampler has filled the current buffer set
  virtual void Post() = 0;  // hands the current buffer set back and moves to the next
  // additions
  virtual bool TimedWait(double seconds) = 0;
  virtual const char *LastError() const = 0;
  // After a wait: when the sampler hands the feature rows over in pieces (a buffer too large to
  // share whole), copies the batch's n_rows rows into one buffer of this process, which
  // GetFloatFeatures then returns.  0, or -1 with the reason in LastError().
  virtual int Assemble(int64_t n_rows) = 0;
};
IPCEnv *NewIPCEnv();

}  // namespace legion_trainer
extern "C" {
#endif

#define LEGION_IPC_MAX_HOPS 3

// What get_next returns in the reference, as plain pointers: ids, features, labels, then
// (agg_src, agg_dst) per block from the LAST hop to the first (ipc_cuda_kernel.cu:194-240).
typedef struct legion_ipc_batch {
  int32_t *ids;       int64_t n_ids;          /* node_counter[9 + hops] */
  void    *features;                          /* [n_ids][feature_dim], row i belongs to ids[i] */
  int32_t *labels;    int64_t n_labels;       /* node_counter[9] */
  int32_t  hop_num;
  int32_t *agg_src[LEGION_IPC_MAX_HOPS];      /* [0] = block of the last hop */
  int32_t *agg_dst[LEGION_IPC_MAX_HOPS];
  int64_t  n_edges[LEGION_IPC_MAX_HOPS];
  int32_t  node_counter[16], edge_counter[16]; /* host copies of the two headers */
} legion_ipc_batch;

int         legion_ipc_initialize(void);                       /* 0, or -1 (see legion_ipc_last_error) */
const char *legion_ipc_last_error(void);
int         legion_ipc_get_next(legion_ipc_batch *out, double wait_seconds);  /* waits, then fills `out` */
int         legion_ipc_get_block_size(int32_t *out, int capacity);  /* (src nodes, dst nodes) per block, last hop first; returns count */
void        legion_ipc_get_steps(int32_t steps[3]);
void        legion_ipc_synchronize(void);                      /* hands the batch's buffers back */
void        legion_ipc_finalize(void);

#ifdef __cplusplus
}
#endif
