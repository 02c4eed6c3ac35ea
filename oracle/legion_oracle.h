/*
 * legion_oracle.h -- CPU oracle of the sampling-server hot path.
 *
 * TEST INFRASTRUCTURE ONLY.  This is the checker the HIP path is compared
 * against; nothing in the shipped library may call it.  Only the test-suite,
 * the smoke check and the cpu_baseline leg of the benchmark load it.
 *
 * Every function is a plain sequential (or trivially loop-parallel) statement
 * of the sampling specification.  The reference (Legion-IBP) fixes semantics,
 * buffer contracts and shapes; the arithmetic that the reference leaves
 * order-dependent or delegates to absent third-party code (thrust::minstd_rand,
 * atomic arrival order, the un-vendored IBP codec, the missing LRU source) is
 * replaced by the deterministic rules stated beside each function below.
 *
 * Pinning status (what independent check fixes each function):
 *   orc_philox4x32_10      Random123 known-answer vectors (3 KATs)
 *   orc_sample_positions   closed forms (deg<=f, deg=0), exact-subset
 *                          enumeration + chi-square over seeds, invariants; for
 *                          deg>f every pick against Floyd's rule stated in plain
 *                          Python on orc_draw words (itself pinned by the KATs)
 *   orc_sample_batch       invariants against a brute-force python pass
 *                          (dict first-occurrence relabel, adjacency membership),
 *                          closed-form counter identities
 *   orc_static_cache_build closed form (rank by degree desc, id asc) checked
 *                          against numpy lexsort
 *   orc_lru_*              trace replay against an independent python
 *                          model + invariants (occupancy, key uniqueness)
 *   orc_quantize/dequant   numpy float32/float16 arithmetic (IEEE, same ops)
 *   orc_f32_to_f16 etc.    numpy.float16 conversion (exhaustive over fp16)
 *   orc_gather_rows        memcmp against numpy fancy indexing
 *   orc_gather_rows_int8   numpy: hits = float32(q) * scale rounded to the row type,
 *                          misses = the host rows, byte for byte
 */
#ifndef LEGION_ORACLE_H
#define LEGION_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ORC_MAX_HOPS 3
#define ORC_F32 0
#define ORC_F16 1

/* ---- RNG ------------------------------------------------------------- */
void     orc_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]);
/* word 0 of Philox(key=(seed lo,hi), ctr=(node,hop,slot,0)) */
uint32_t orc_draw(uint64_t seed, uint32_t hop, uint32_t node, uint32_t slot);

/* ---- sampling -------------------------------------------------------- */
/* positions (0-based, inside the CSR row) chosen for one node; returns count */
int32_t orc_sample_positions(uint64_t seed, int32_t hop, int32_t node, int64_t deg,
                             int32_t fanout, int64_t *pos_out);

/* One mini-batch: multi-hop sample + first-occurrence dedup/relabel.
 * blk_indptr holds the per-hop block CSR row pointers back to back: hop k
 * (1-based) occupies n_{k-1}+1 entries.  Returns 0, or <0 on capacity error. */
int orc_sample_batch(const int64_t *indptr, const int32_t *indices, int64_t n_nodes,
                     const int32_t *seeds, int32_t n_seeds,
                     const int32_t *fanout, int32_t hops, uint64_t seed,
                     int32_t *ids, int64_t ids_cap,
                     int32_t *agg_src_ids, int32_t *agg_src_off, int32_t *agg_dst_off,
                     int64_t edge_cap,
                     int32_t *blk_indptr, int64_t blk_indptr_cap,
                     int32_t node_counter[16], int32_t edge_counter[16],
                     int threads);

/* ---- static hot-set cache ------------------------------------------- */
/* slot_of[v] = slot (0..cap-1) if v is cached else -1 */
void orc_static_cache_build(const int64_t *indptr, int64_t n_nodes, int64_t cap_rows,
                            int32_t *slot_of);

/* the same with an arbitrary ranking key per node (e.g. presampling counts) */
void orc_static_cache_build_keys(const int64_t *keys, int64_t n_nodes, int64_t cap_rows,
                                 int32_t *slot_of);

/* ---- LRU dynamic cache ---------------------------------------------- */
void *orc_lru_create(int64_t n_sets, int32_t ways, int64_t row_bytes);
void  orc_lru_destroy(void *lru);
/* One batch.  hit_slot[i] = slot or -1 (state before the batch);
 * fill_slot[i] = slot a missing id was inserted into, or -1.  An id that appears
 * more than once in the batch is inserted once, by its first position.
 * If host_rows/out are non-null, also gathers: hits from the cache's own row
 * store, misses from host_rows, and copies inserted rows into the store.  The
 * store (n_sets * ways * row_bytes) is only allocated by the first call that
 * brings host_rows; use either every call with host_rows or none. */
void  orc_lru_access(void *lru, const int32_t *ids, int64_t n,
                     int32_t *hit_slot, int32_t *fill_slot,
                     const void *host_rows, void *out);
void  orc_lru_state(void *lru, int32_t *keys, int32_t *last_use);

/* ---- int8 codec ------------------------------------------------------ */
uint16_t orc_f32_to_f16(float x);
float    orc_f16_to_f32(uint16_t h);
void orc_quantize_rows(const void *rows, int32_t dtype, int64_t n_rows, int32_t dim,
                       int8_t *q, float *scale);
void orc_dequant_rows(const int8_t *q, const float *scale, int64_t n_rows, int32_t dim,
                      void *out, int32_t out_dtype);

/* ---- gather ---------------------------------------------------------- */
/* out[i] = slot[i] >= 0 ? cache_rows[slot[i]] : host_rows[ids[i]]  (byte copy) */
void orc_gather_rows(const int32_t *ids, const int32_t *slot, int64_t n,
                     const void *cache_rows, const void *host_rows, int64_t row_bytes,
                     void *out, int threads);
/* int8 cache: hit -> dequantised row, miss -> raw host row (dtype = out dtype) */
void orc_gather_rows_int8(const int32_t *ids, const int32_t *slot, int64_t n,
                          const int8_t *q_rows, const float *scales,
                          const void *host_rows, int32_t dim, int32_t dtype,
                          void *out, int threads);

/* ---- synthetic graph (same integer arithmetic as the device generator) */
void orc_synth_degrees(uint64_t seed, const uint32_t *cdf, int32_t cdf_len,
                       int64_t n_nodes, int64_t *indptr /* n_nodes+1 */);
void orc_synth_indices(uint64_t seed, const int64_t *indptr, int64_t n_nodes,
                       int32_t mode /*0 uniform, 1 degree-proportional*/,
                       int32_t *indices, int threads);
void orc_synth_trainset(uint64_t seed, int64_t n_nodes, int32_t n_train, int32_t *ids);

#ifdef __cplusplus
}
#endif
#endif
