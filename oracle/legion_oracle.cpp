/*
 * legion_oracle.cpp -- CPU oracle of the sampling-server hot path.
 *
 * TEST INFRASTRUCTURE ONLY (see legion_oracle.h).  Sequential statements of the
 * specification; the only parallelism is "#pragma omp parallel for" over loops
 * whose iterations are independent by construction, so results never depend on
 * the thread count.
 *
 * Reference files whose SEMANTICS this follows (paths relative to the
 * Legion-IBP tree):
 *   sampling_server/src/engine/operator_impl.cu:28-56    seed staging
 *   sampling_server/src/engine/operator_impl.cu:58-91    16-int counter headers
 *   sampling_server/src/engine/operator_impl.cu:178-302  hop semantics
 *   sampling_server/src/engine/operator_impl.cu:304-317  relabel to local ids
 *   sampling_server/src/cache/cache_impl.cuh:239-303     gather hit/miss addressing
 *   sampling_server/src/comp_cache/static_cache_kernel.cuh:6-29,185-266
 *                                                        set-associative addressing
 * Build: g++ -O3 -ffp-contract=off -fno-fast-math (no FMA contraction, so the
 * int8 codec rounds exactly like the device code).
 */
#include "legion_oracle.h"

#include <algorithm>
#include <cmath>
#include <cstring>
#include <numeric>
#include <unordered_map>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

namespace {

/* ------------------------------------------------------------------ RNG */
/* Philox4x32-10 (Salmon et al., SC'11).  Replaces the reference's
 * thrust::minstd_rand, which is re-created with the default seed for every
 * node (operator_impl.cu:244-246) and therefore never varies. */
constexpr uint32_t PHILOX_M0 = 0xD2511F53u, PHILOX_M1 = 0xCD9E8D57u;
constexpr uint32_t PHILOX_W0 = 0x9E3779B9u, PHILOX_W1 = 0xBB67AE85u;

inline void philox(const uint32_t c_in[4], const uint32_t k_in[2], uint32_t out[4]) {
  uint32_t c0 = c_in[0], c1 = c_in[1], c2 = c_in[2], c3 = c_in[3];
  uint32_t k0 = k_in[0], k1 = k_in[1];
  for (int r = 0; r < 10; ++r) {
    uint64_t p0 = (uint64_t)PHILOX_M0 * c0;
    uint64_t p1 = (uint64_t)PHILOX_M1 * c2;
    uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    uint32_t n1 = (uint32_t)p1;
    uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += PHILOX_W0; k1 += PHILOX_W1;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

inline uint32_t draw(uint64_t seed, uint32_t hop, uint32_t node, uint32_t slot) {
  uint32_t c[4] = {node, hop, slot, 0u};
  uint32_t k[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  uint32_t o[4];
  philox(c, k, o);
  return o[0];
}

inline uint32_t mulhi32(uint32_t a, uint32_t b) { return (uint32_t)(((uint64_t)a * b) >> 32); }
inline uint64_t mulhi64(uint64_t a, uint64_t b) {
  return (uint64_t)(((unsigned __int128)a * b) >> 64);
}

/* ------------------------------------------------------- pick positions */
/* deg <= fanout: the whole row in CSR order (kept from operator_impl.cu:241-242).
 * deg  > fanout: Floyd's sampling without replacement over row positions,
 *   s = 0..f-1:  j = deg-f+s,  t = floor(draw(s) * (j+1) / 2^32),
 *                pick_s = (t already picked) ? j : t
 * which is exactly uniform over f-subsets; replaces the 10-try redraw of
 * operator_impl.cu:247-258 that may leave duplicates. */
int32_t sample_positions(uint64_t seed, int32_t hop, int32_t node, int64_t deg, int32_t f,
                         int64_t *pos) {
  if (deg <= 0 || f <= 0) return 0;
  if (deg <= f) {
    for (int64_t s = 0; s < deg; ++s) pos[s] = s;
    return (int32_t)deg;
  }
  for (int32_t s = 0; s < f; ++s) {
    uint32_t j = (uint32_t)(deg - f + s);
    uint32_t t = mulhi32(draw(seed, (uint32_t)hop, (uint32_t)node, (uint32_t)s), j + 1u);
    bool seen = false;
    for (int32_t q = 0; q < s; ++q) seen |= (pos[q] == (int64_t)t);
    pos[s] = seen ? (int64_t)j : (int64_t)t;
  }
  return f;
}

/* -------------------------------------------------------- fp16 <-> fp32 */
inline float f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu, man = h & 0x3FFu, bits;
  if (exp == 0) {
    if (man == 0) bits = sign;
    else {                                   /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; ++e; } while (!(man & 0x400u));
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3FFu) << 13);
    }
  } else if (exp == 31) bits = sign | 0x7F800000u | (man << 13);
  else bits = sign | ((exp + 112u) << 23) | (man << 13);
  float f; std::memcpy(&f, &bits, 4); return f;
}

/* round-to-nearest-even, like the device's v_cvt_f16_f32 */
inline uint16_t f32_to_f16(float x) {
  uint32_t b; std::memcpy(&b, &x, 4);
  uint32_t sign = (b >> 16) & 0x8000u;
  uint32_t a = b & 0x7FFFFFFFu;
  if (a >= 0x7F800000u) return (uint16_t)(sign | 0x7C00u | (a > 0x7F800000u ? 0x200u | ((a >> 13) & 0x3FFu) : 0u));
  if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u);        /* >= 65520 -> inf */
  if (a < 0x33000001u) return (uint16_t)sign;                      /* <= 2^-25 -> 0 */
  int32_t e = (int32_t)(a >> 23) - 127;
  uint32_t m = (a & 0x7FFFFFu) | 0x800000u;                        /* 24-bit significand */
  int shift = (e < -14) ? (13 + (-14 - e)) : 13;                   /* bits dropped */
  uint32_t kept = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1);
  if (rem > half || (rem == half && (kept & 1u))) ++kept;
  uint32_t h;
  if (e < -14) h = kept;                                            /* subnormal (may carry into normal) */
  else h = ((uint32_t)(e + 15) << 10) + (kept - 0x400u);            /* carry propagates into exponent */
  return (uint16_t)(sign | h);
}

struct Lru {
  int64_t sets; int32_t ways; int64_t row_bytes; int32_t tick;
  std::vector<int32_t> keys, last_use;
  std::vector<uint8_t> rows;
};

}  // namespace

extern "C" {

void orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  philox(ctr, key, out);
}
uint32_t orc_draw(uint64_t seed, uint32_t hop, uint32_t node, uint32_t slot) {
  return draw(seed, hop, node, slot);
}
int32_t orc_sample_positions(uint64_t seed, int32_t hop, int32_t node, int64_t deg,
                             int32_t fanout, int64_t *pos_out) {
  return sample_positions(seed, hop, node, deg, fanout, pos_out);
}

/* One mini-batch.
 *  - seeds keep local ids 0..B-1 in caller order (operator_impl.cu:52); a seed
 *    value that occurs twice keeps both rows, later lookups resolve to the first.
 *  - hop k (0-based) samples from ALL n_k nodes known so far, in local-id order
 *    (operator_impl.cu:206), fanout[k] per node; edge order = (node, slot).
 *  - edge direction: src = sampled neighbour, dst = the node it was sampled for
 *    (operator_impl.cu:196,284-285).
 *  - a neighbour not seen before gets the next local id in edge order
 *    (first occurrence); replaces the atomic arrival order of :266-293.
 *  - headers as counter_update leaves them after the last hop (:58-91):
 *    node_counter[8]=hops, [9+k]=#nodes after hop k (k=0 is the seed count),
 *    [0]/[1]=offset/size of the last frontier, [7]=total, [2..5] mirror [0],[1];
 *    edge_counter[9+k]=#edges of hop k, [12+k]=first edge of hop k (k=1..hops),
 *    [0]=first edge of the last hop, [1]=its size.
 */
int orc_sample_batch(const int64_t *indptr, const int32_t *indices, int64_t n_nodes,
                     const int32_t *seeds, int32_t n_seeds,
                     const int32_t *fanout, int32_t hops, uint64_t seed,
                     int32_t *ids, int64_t ids_cap,
                     int32_t *agg_src_ids, int32_t *agg_src_off, int32_t *agg_dst_off,
                     int64_t edge_cap,
                     int32_t *blk_indptr, int64_t blk_indptr_cap,
                     int32_t node_counter[16], int32_t edge_counter[16],
                     int threads) {
  if (hops < 1 || hops > ORC_MAX_HOPS || n_seeds < 0 || n_seeds > ids_cap) return -1;
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
  std::memset(node_counter, 0, 16 * sizeof(int32_t));
  std::memset(edge_counter, 0, 16 * sizeof(int32_t));
  std::unordered_map<int32_t, int32_t> local;     /* global id -> local id */
  local.reserve((size_t)n_seeds * 4);
  for (int32_t i = 0; i < n_seeds; ++i) {
    if (seeds[i] < 0 || seeds[i] >= n_nodes) return -2;
    ids[i] = seeds[i];
    local.emplace(seeds[i], i);                    /* first occurrence wins */
  }
  int64_t n_prev = n_seeds, e_off = 0, ip_off = 0;
  node_counter[8] = hops;
  node_counter[9] = n_seeds;
  std::vector<int64_t> row_off;
  for (int32_t k = 0; k < hops; ++k) {
    const int32_t f = fanout[k];
    if (f < 0) return -1;
    /* per-node output counts are known before sampling: min(deg, f) */
    row_off.assign((size_t)n_prev + 1, 0);
    for (int64_t i = 0; i < n_prev; ++i) {
      int64_t deg = indptr[ids[i] + 1] - indptr[ids[i]];
      row_off[i + 1] = row_off[i] + std::min<int64_t>(deg, f);
    }
    const int64_t e_k = row_off[n_prev];
    if (e_off + e_k > edge_cap || ip_off + n_prev + 1 > blk_indptr_cap) return -3;
    for (int64_t i = 0; i <= n_prev; ++i) blk_indptr[ip_off + i] = (int32_t)row_off[i];
#pragma omp parallel
    {
      std::vector<int64_t> pos((size_t)std::max(f, 1));
#pragma omp for schedule(dynamic, 256)
      for (int64_t i = 0; i < n_prev; ++i) {
        const int32_t v = ids[i];
        const int64_t beg = indptr[v], deg = indptr[v + 1] - beg;
        int32_t c = sample_positions(seed, k, v, deg, f, pos.data());
        for (int32_t s = 0; s < c; ++s) {
          agg_src_ids[e_off + row_off[i] + s] = indices[beg + pos[s]];
          agg_dst_off[e_off + row_off[i] + s] = (int32_t)i;
        }
      }
    }
    /* first-occurrence relabel, strictly in edge order */
    int64_t n_now = n_prev;
    for (int64_t e = 0; e < e_k; ++e) {
      const int32_t g = agg_src_ids[e_off + e];
      auto it = local.find(g);
      int32_t l;
      if (it == local.end()) {
        if (n_now >= ids_cap) return -3;
        l = (int32_t)n_now;
        ids[n_now++] = g;
        local.emplace(g, l);
      } else l = it->second;
      agg_src_off[e_off + e] = l;
    }
    node_counter[9 + k + 1] = (int32_t)n_now;
    edge_counter[9 + k + 1] = (int32_t)e_k;
    edge_counter[12 + k + 1] = (int32_t)e_off;
    node_counter[0] = (int32_t)n_prev;
    node_counter[1] = (int32_t)(n_now - n_prev);
    edge_counter[0] = (int32_t)e_off;
    edge_counter[1] = (int32_t)e_k;
    ip_off += n_prev + 1;
    e_off += e_k;
    n_prev = n_now;
  }
  node_counter[7] = (int32_t)n_prev;
  node_counter[2] = node_counter[4] = node_counter[0];
  node_counter[3] = node_counter[5] = node_counter[1];
  return 0;
}

/* Static hot-set membership: v is cached iff its rank under
 * (out-degree descending, id ascending) is < cap_rows; the slot of a cached
 * node is the number of cached nodes with a smaller id.  Replaces presampled
 * hotness + an unstable device sort (cache/cache.cu:354-447), whose tie order
 * is undefined. */
void orc_static_cache_build(const int64_t *indptr, int64_t n_nodes, int64_t cap_rows,
                            int32_t *slot_of) {
  std::vector<int64_t> deg((size_t)n_nodes);
  for (int64_t v = 0; v < n_nodes; ++v) deg[v] = indptr[v + 1] - indptr[v];
  orc_static_cache_build_keys(deg.data(), n_nodes, cap_rows, slot_of);
}

/* The same selection for any ranking key (key descending, id ascending); with
 * key = presampling appearance counts this is the reference's hot-set policy
 * (cache/cache.cu:354-447) with its undefined tie order made definite. */
void orc_static_cache_build_keys(const int64_t *keys, int64_t n_nodes, int64_t cap_rows,
                                 int32_t *slot_of) {
  std::vector<int32_t> order((size_t)n_nodes);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) { return keys[a] > keys[b]; });
  for (int64_t v = 0; v < n_nodes; ++v) slot_of[v] = -1;
  const int64_t cap = std::min(std::max<int64_t>(cap_rows, 0), n_nodes);
  for (int64_t r = 0; r < cap; ++r) slot_of[order[r]] = 0;
  int32_t next = 0;
  for (int64_t v = 0; v < n_nodes; ++v)
    if (slot_of[v] == 0) slot_of[v] = next++;
}

/* LRU dynamic cache, batch-synchronous.  Table shape follows the reference's
 * set-associative StaticCache (set = id mod n_sets, ways contiguous;
 * comp_cache/static_cache_kernel.cuh:6-9,185-231); the eviction policy is ours
 * because the reference's DynamicCache source is absent from its tree:
 *   1. every id of batch t is looked up in the state left by batch t-1;
 *      a hit sets last_use = t;
 *   2. the misses, in the order given, each take the way of their set with the
 *      smallest (last_use, way) among ways with last_use < t (empty ways have
 *      last_use 0); the taken way gets last_use = t; if no way qualifies the id
 *      is not cached.
 * ids within a batch are distinct (they come out of the dedup). */
void *orc_lru_create(int64_t n_sets, int32_t ways, int64_t row_bytes) {
  Lru *c = new Lru;
  c->sets = n_sets; c->ways = ways; c->row_bytes = row_bytes; c->tick = 0;
  c->keys.assign((size_t)(n_sets * ways), -1);
  c->last_use.assign((size_t)(n_sets * ways), 0);
  return c;  // the row store is set up by the first access that brings host rows
}
void orc_lru_destroy(void *lru) { delete (Lru *)lru; }

void orc_lru_access(void *lru, const int32_t *ids, int64_t n, int32_t *hit_slot,
                    int32_t *fill_slot, const void *host_rows, void *out) {
  Lru *c = (Lru *)lru;
  const int32_t t = ++c->tick;
  const int64_t rb = c->row_bytes;
  // policy-only use (host_rows == NULL) never pays for sets * ways * row_bytes of rows
  if (host_rows && c->rows.empty()) c->rows.assign((size_t)(c->sets * c->ways * rb), 0);
  for (int64_t i = 0; i < n; ++i) {
    const int64_t base = ((int64_t)ids[i] % c->sets) * c->ways;
    hit_slot[i] = -1;
    for (int32_t w = 0; w < c->ways; ++w)
      if (c->keys[base + w] == ids[i]) { hit_slot[i] = (int32_t)(base + w); c->last_use[base + w] = t; }
    if (out && host_rows) {
      const uint8_t *src = hit_slot[i] >= 0 ? c->rows.data() + (int64_t)hit_slot[i] * rb
                                            : (const uint8_t *)host_rows + (int64_t)ids[i] * rb;
      std::memcpy((uint8_t *)out + i * rb, src, (size_t)rb);
    }
  }
  for (int64_t i = 0; i < n; ++i) {
    fill_slot[i] = -1;
    if (hit_slot[i] >= 0) continue;
    const int64_t base = ((int64_t)ids[i] % c->sets) * c->ways;
    bool placed = false;  // an id that appears twice in the batch (a repeated seed) is inserted once
    for (int32_t w = 0; w < c->ways; ++w) placed = placed || c->keys[base + w] == ids[i];
    if (placed) continue;
    int32_t best = -1;
    for (int32_t w = 0; w < c->ways; ++w)
      if (c->last_use[base + w] < t && (best < 0 || c->last_use[base + w] < c->last_use[base + best]))
        best = w;
    if (best < 0) continue;
    c->keys[base + best] = ids[i];
    c->last_use[base + best] = t;
    fill_slot[i] = (int32_t)(base + best);
    if (host_rows)
      std::memcpy(c->rows.data() + (base + best) * rb,
                  (const uint8_t *)host_rows + (int64_t)ids[i] * rb, (size_t)rb);
  }
}
void orc_lru_state(void *lru, int32_t *keys, int32_t *last_use) {
  Lru *c = (Lru *)lru;
  std::memcpy(keys, c->keys.data(), c->keys.size() * 4);
  std::memcpy(last_use, c->last_use.data(), c->last_use.size() * 4);
}

/* int8 codec (replaces the lossless IBP bit-plane codec whose source is not in
 * the reference tree, comp_cache/compress_cache_kernel.cuh:5-7):
 *   a = max_i |x_i| (fp16 inputs widened exactly), scale = a / 127,
 *   q_i = clamp(rint(x_i / scale), -127, 127)   (a == 0: scale = 0, q = 0)
 *   y_i = float(q_i) * scale   -- one IEEE multiply, then RNE to the out dtype. */
uint16_t orc_f32_to_f16(float x) { return f32_to_f16(x); }
float orc_f16_to_f32(uint16_t h) { return f16_to_f32(h); }

void orc_quantize_rows(const void *rows, int32_t dtype, int64_t n_rows, int32_t dim,
                       int8_t *q, float *scale) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n_rows; ++r) {
    float a = 0.0f;
    for (int32_t i = 0; i < dim; ++i) {
      float x = dtype == ORC_F16 ? f16_to_f32(((const uint16_t *)rows)[r * dim + i])
                                 : ((const float *)rows)[r * dim + i];
      a = std::max(a, std::fabs(x));
    }
    volatile float sc = a / 127.0f;
    scale[r] = sc;
    for (int32_t i = 0; i < dim; ++i) {
      float x = dtype == ORC_F16 ? f16_to_f32(((const uint16_t *)rows)[r * dim + i])
                                 : ((const float *)rows)[r * dim + i];
      float v = (a == 0.0f) ? 0.0f : std::nearbyintf(x / sc);
      v = std::min(127.0f, std::max(-127.0f, v));
      q[r * dim + i] = (int8_t)v;
    }
  }
}

void orc_dequant_rows(const int8_t *q, const float *scale, int64_t n_rows, int32_t dim,
                      void *out, int32_t out_dtype) {
#pragma omp parallel for schedule(static)
  for (int64_t r = 0; r < n_rows; ++r)
    for (int32_t i = 0; i < dim; ++i) {
      volatile float y = (float)q[r * dim + i] * scale[r];
      if (out_dtype == ORC_F16) ((uint16_t *)out)[r * dim + i] = f32_to_f16(y);
      else ((float *)out)[r * dim + i] = y;
    }
}

/* Gather (cache/cache_impl.cuh:239-303): row i of the output belongs to ids[i];
 * hit -> cache row `slot`, miss -> host row `id` (the reference's `id % N` is a
 * no-op for valid ids). */
void orc_gather_rows(const int32_t *ids, const int32_t *slot, int64_t n,
                     const void *cache_rows, const void *host_rows, int64_t row_bytes,
                     void *out, int threads) {
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    const uint8_t *src = (slot && slot[i] >= 0)
                             ? (const uint8_t *)cache_rows + (int64_t)slot[i] * row_bytes
                             : (const uint8_t *)host_rows + (int64_t)ids[i] * row_bytes;
    std::memcpy((uint8_t *)out + i * row_bytes, src, (size_t)row_bytes);
  }
}

void orc_gather_rows_int8(const int32_t *ids, const int32_t *slot, int64_t n,
                          const int8_t *q_rows, const float *scales,
                          const void *host_rows, int32_t dim, int32_t dtype,
                          void *out, int threads) {
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
  const int64_t esz = dtype == ORC_F16 ? 2 : 4;
#pragma omp parallel for schedule(static)
  for (int64_t i = 0; i < n; ++i) {
    uint8_t *dst = (uint8_t *)out + i * dim * esz;
    if (slot[i] >= 0)
      orc_dequant_rows(q_rows + (int64_t)slot[i] * dim, scales + slot[i], 1, dim, dst, dtype);
    else
      std::memcpy(dst, (const uint8_t *)host_rows + (int64_t)ids[i] * dim * esz, (size_t)(dim * esz));
  }
}

/* Synthetic power-law graph; pure integer arithmetic on Philox words so the
 * device generator reproduces it bit for bit.
 *  degree(v)  = first j with u <= cdf[j], u = Philox(seed; v_lo, v_hi, 0x5eed0001, 0).w0
 *  indices[e] = mode 0: floor(x * N / 2^64)
 *               mode 1: owner of edge slot floor(x * E / 2^64)  (degree-proportional)
 *               x = 64 bits of Philox(seed; e_lo, e_hi, 0x5eed0002, 0)
 */
void orc_synth_degrees(uint64_t seed, const uint32_t *cdf, int32_t cdf_len, int64_t n_nodes,
                       int64_t *indptr) {
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  indptr[0] = 0;
  for (int64_t v = 0; v < n_nodes; ++v) {
    uint32_t c[4] = {(uint32_t)v, (uint32_t)((uint64_t)v >> 32), 0x5eed0001u, 0u}, o[4];
    philox(c, key, o);
    int64_t d = std::lower_bound(cdf, cdf + cdf_len, o[0]) - cdf;
    if (d >= cdf_len) d = cdf_len - 1;
    indptr[v + 1] = indptr[v] + d;
  }
}

void orc_synth_indices(uint64_t seed, const int64_t *indptr, int64_t n_nodes, int32_t mode,
                       int32_t *indices, int threads) {
#ifdef _OPENMP
  if (threads > 0) omp_set_num_threads(threads);
#else
  (void)threads;
#endif
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  const int64_t n_edges = indptr[n_nodes];
#pragma omp parallel for schedule(static)
  for (int64_t e = 0; e < n_edges; ++e) {
    uint32_t c[4] = {(uint32_t)e, (uint32_t)((uint64_t)e >> 32), 0x5eed0002u, 0u}, o[4];
    philox(c, key, o);
    uint64_t x = (uint64_t)o[0] | ((uint64_t)o[1] << 32);
    if (mode == 0) indices[e] = (int32_t)mulhi64(x, (uint64_t)n_nodes);
    else {
      int64_t slot = (int64_t)mulhi64(x, (uint64_t)n_edges);
      indices[e] = (int32_t)(std::upper_bound(indptr, indptr + n_nodes + 1, slot) - indptr - 1);
    }
  }
}

/* n_train distinct ids: stratum p = (i * P) mod n_train (P coprime with n_train)
 * covers [p*stride, (p+1)*stride); the id is a Philox-uniform point inside it. */
void orc_synth_trainset(uint64_t seed, int64_t n_nodes, int32_t n_train, int32_t *ids) {
  uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  const uint32_t stride = (uint32_t)(n_nodes / n_train);
  uint64_t P = 1000003;
  while (std::gcd<uint64_t, uint64_t>(P, (uint64_t)n_train) != 1) ++P;
  for (int32_t i = 0; i < n_train; ++i) {
    uint32_t p = (uint32_t)(((uint64_t)i * P) % (uint64_t)n_train);
    uint32_t c[4] = {p, 0u, 0x5eed0003u, 0u}, o[4];
    philox(c, key, o);
    ids[i] = (int32_t)(p * stride + mulhi32(o[0], stride));
  }
}

}  // extern "C"
