// Device-side building blocks: Philox4x32-10, open-addressing probes, wave64 /
// block scans.  gfx950 only (64-wide wavefronts).
#pragma once

#include "common.hpp"
#include "lookback.hpp"

namespace lmi {

// ------------------------------------------------------------------ Philox
// Philox4x32-10 (Salmon et al. 2011); constants as published.
struct Philox4 {
  uint32_t x, y, z, w;
};

__device__ __forceinline__ Philox4 philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                                 uint32_t k0, uint32_t k1) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    c0 = hi1 ^ c1 ^ k0;
    c1 = lo1;
    c2 = hi0 ^ c3 ^ k1;
    c3 = lo0;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return Philox4{c0, c1, c2, c3};
}

// The sampler's draw: key = 64-bit batch seed, counter = (node, hop, slot, 0).
__device__ __forceinline__ uint32_t sample_draw(uint64_t seed, uint32_t hop, uint32_t node,
                                                uint32_t slot) {
  return philox4x32_10(node, hop, slot, 0u, (uint32_t)seed, (uint32_t)(seed >> 32)).x;
}

// ------------------------------------------------------------------ faults
// A condition the host must hear about: recorded in the batch state (read back by
// lmi_batch_counters) and in the server's sticky fault word, which lives in pinned host
// memory and is never cleared by a later batch, so the host sees it without reading the
// device (lmi_server_status).
__device__ __forceinline__ void raise_fault(DevState *st, int which) {
  if (which == kFaultBadId) st->bad_id = 1; else st->scan_fault = 1;
  if (st->fault) __hip_atomic_store(&st->fault[which], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// -------------------------------------------------------------- hash table
__device__ __forceinline__ uint32_t hash_id(int32_t key, int log2cap) {
  return ((uint32_t)key * 0x9E3779B1u) >> (32 - log2cap);
}

// A stored key is `key | tag`: the tag (an epoch number in the bits above the widest id)
// says which batch wrote the slot.  A slot whose tag bits differ from the current tag is
// free -- never written (key -1: every tag bit set) or left by an earlier batch -- so the
// table needs no clearing between batches until the epochs run out.  Untagged tables use
// tag 0 with the sign bit as mask: only the empty key -1 is free.
// Insert `key` (if absent) and lower its value to min(value, cand); returns the
// slot index.  One 8-byte load reads key and value together; a free slot is claimed
// with one 8-byte compare-and-swap that writes key and value at once.  Within a batch
// a slot only ever goes free -> key, so a stale non-free read is still correct and a
// stale free read is resolved by the CAS.  Values only ever decrease, so a stale value
// is never too low: when the value read is already <= cand the atomic can be skipped,
// which removes almost all same-address atomics on frequently sampled hub nodes.
// The slot index comes back with kKnownRepeat set when the insert already saw a lower
// value: such a candidate is certainly not the key's first occurrence, and whoever asks
// later need not read the slot to learn that.  (Without the bit it may or may not be.)
constexpr uint32_t kKnownRepeat = 0x80000000u;
__device__ __forceinline__ uint32_t table_insert_min(HashSlot *slots, int log2cap, int32_t key, int32_t cand,
                                                     int32_t tag = 0, int32_t tag_mask = kUntaggedMask) {
  const uint32_t mask = (1u << log2cap) - 1u;
  const int32_t stored = key | tag;
  uint32_t h = hash_id(key, log2cap);
  while (true) {
    unsigned long long *word = reinterpret_cast<unsigned long long *>(&slots[h]);
    const unsigned long long raw = *reinterpret_cast<const volatile unsigned long long *>(word);
    const int32_t k = (int32_t)(uint32_t)raw, v = (int32_t)(uint32_t)(raw >> 32);
    if ((k & tag_mask) != tag) {  // free: claim it with key and value together
      const unsigned long long mine = (unsigned long long)(uint32_t)stored | ((unsigned long long)(uint32_t)cand << 32);
      if (atomicCAS(word, raw, mine) == raw) return h;
      continue;  // somebody else took it: look at what it holds now
    }
    if (k == stored) {
      if (v > cand) {
        atomicMin(&slots[h].val, cand);
        return h;
      }
      return h | kKnownRepeat;  // a lower candidate is already there: this one cannot be the minimum
    }
    h = (h + 1) & mask;
  }
}

// Read-only probe: value or -1.
__device__ __forceinline__ int32_t table_find(const HashSlot *slots, int log2cap, int32_t key, int32_t tag = 0,
                                              int32_t tag_mask = kUntaggedMask) {
  const uint32_t mask = (1u << log2cap) - 1u;
  const int32_t stored = key | tag;
  uint32_t h = hash_id(key, log2cap);
  while (true) {
    const int2 kv = *reinterpret_cast<const int2 *>(&slots[h]);
    if (kv.x == stored) return kv.y;
    if ((kv.x & tag_mask) != tag) return -1;
    h = (h + 1) & mask;
  }
}

// Last step of a hop: the local id of every edge source is the value its table slot
// holds once the hop's first occurrences have published theirs.  Strided over the
// `n_threads` threads that take part, `tid` being this thread's place among them.
struct FillArgs {
  const DevState *st;
  const HashSlot *slots;
  const int32_t *eslot;  // table slot per edge of hop `hop` (| kKnownRepeat)
  int32_t *agg_src_off;
  int hop;               // -1: nothing to fill
};

__device__ __forceinline__ void fill_local_ids(const FillArgs &f, int64_t tid, int64_t n_threads) {
  if (f.hop < 0) return;
  const int n = f.st->edge_counter[9 + f.hop + 1];
  const int eoff = f.st->edge_counter[12 + f.hop + 1];
  // four edges in flight per thread: the two dependent reads of each overlap those of the others
  for (int64_t e = tid; e < n; e += 4 * n_threads) {
    int32_t slot[4], val[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) slot[u] = (e + u * n_threads < n) ? (f.eslot[e + u * n_threads] & (int32_t)~kKnownRepeat) : 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) val[u] = (e + u * n_threads < n) ? f.slots[slot[u]].val : 0;
#pragma unroll
    for (int u = 0; u < 4; ++u)
      if (e + u * n_threads < n) f.agg_src_off[eoff + e + u * n_threads] = val[u];
  }
}

// A launch that serves n pipes interleaves them over blockIdx.x (grid_row).
#define LMI_GRID_ROW(n_rows)                                                   \
  const GridRow lmi_gr_ = grid_row(blockIdx.x, (unsigned)(n_rows));            \
  const int row = lmi_gr_.row;                                                 \
  const int bx = lmi_gr_.bx;                                                   \
  const int gx = (int)(gridDim.x / (unsigned)(n_rows));                        \
  (void)gx

// ------------------------------------------------------------------- scans
__device__ __forceinline__ int wave_inclusive_scan(int v) {
  const int lane = threadIdx.x & (kWave - 1);
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const int t = __shfl_up(v, d, kWave);
    if (lane >= d) v += t;
  }
  return v;
}

// Exclusive scan over a block of BLOCK threads; `total` = sum over the block.
// lds must hold BLOCK / 64 + 1 ints.  Contains __syncthreads: call uniformly.
template <int BLOCK>
__device__ __forceinline__ int block_exclusive_scan(int v, int *lds, int &total) {
  constexpr int NW = BLOCK / kWave;
  const int lane = threadIdx.x & (kWave - 1), wid = threadIdx.x / kWave;
  const int inc = wave_inclusive_scan(v);
  if (lane == kWave - 1) lds[wid] = inc;
  __syncthreads();
  if (wid == 0) {
    int w = (lane < NW) ? lds[lane] : 0;
    const int winc = wave_inclusive_scan(w);
    if (lane < NW) lds[lane] = winc - w;
    if (lane == NW - 1) lds[NW] = winc;
  }
  __syncthreads();
  const int res = inc - v + lds[wid];
  total = lds[NW];
  __syncthreads();
  return res;
}

__device__ __forceinline__ uint64_t lanemask_lt() {
  const int lane = threadIdx.x & (kWave - 1);
  return (lane == 0) ? 0ull : (~0ull >> (kWave - lane));
}

}  // namespace lmi
