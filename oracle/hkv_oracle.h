/*
 * TEST INFRASTRUCTURE ONLY.  CPU restatement (plain C) of the reference's
 * bucketed hash-table algorithm, used as the checker in tests, in the smoke
 * test and as the `cpu_baseline` leg of the benchmark.  Nothing in the shipped
 * library links, loads or calls this file.
 *
 * All pointers are host pointers.  The function set mirrors include/hkv_c_api.h
 * one to one (hkvo_X checks hkv_X).  Every function processes its batch
 * sequentially in input order, which is one of the interleavings the
 * reference's concurrent kernels may produce; under the preconditions the
 * parity tests guarantee (unique keys per batch, pairwise distinct scores, no
 * key re-scored downwards) every interleaving gives the same table.
 *
 * Parity pins (what each part was checked against before being trusted) are
 * listed in the header comment of hkv_oracle.c.
 */
#ifndef HKV_ORACLE_H_
#define HKV_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#include "hkv_c_api.h"

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hkvo_table hkvo_table;

/* utils.cuh:127-135 */
uint64_t hkvo_murmur3_fmix64(uint64_t key);
/* types.cuh:80-109: derive the sentinel keys and masks for a start bit.
 * out[0..6] = empty, reclaim, locked, reserved_mask1, reserved_mask2,
 * vacant_mask1, vacant_mask2.  Returns 0, or -1 if start_bit is out of range. */
int hkvo_reserved_keys(int start_bit, uint64_t out[7]);
/* kernel_utils.cuh:626-643 + :84-96: bucket, start slot and digest of a key for
 * a table with `buckets_num` buckets of 128 slots. */
void hkvo_locate(uint64_t key, uint64_t buckets_num, uint64_t* bkt,
                 uint32_t* start, uint8_t* digest);

/* dual-bucket mode (TableMode::kMemory): both candidate buckets, their start
 * positions and the digest (hash bits 56..63), dual_bucket_utils.cuh:36-74,
 * dual_bucket_upsert.cuh:86-101 */
void hkvo_locate_dual(uint64_t key, uint64_t buckets_num, uint64_t bkt[2],
                      uint32_t start[2], uint8_t* digest);

/* create_table (core_kernels.cuh:327-381) + argument checks of
 * HashTable::init (merlin_hashtable.cuh:1016-1048).  `hybrid_refusal` selects
 * the `score <= min` refusal rule of the hybrid kernels (upsert.cuh:1524)
 * instead of `score < min` (upsert.cuh:188). */
int hkvo_create(const hkv_options* opts, int hybrid_refusal, hkvo_table** out);
void hkvo_destroy(hkvo_table* t);
const char* hkvo_last_error(void);

int hkvo_set_global_epoch(hkvo_table* t, uint64_t epoch);
int hkvo_set_clock(hkvo_table* t, int mode, uint64_t base);

int hkvo_insert_or_assign(hkvo_table* t, uint64_t n, const uint64_t* keys,
                          const void* values, const uint64_t* scores,
                          int ignore_evict_strategy);
int hkvo_insert_and_evict(hkvo_table* t, uint64_t n, const uint64_t* keys,
                          const void* values, const uint64_t* scores,
                          uint64_t* evicted_keys, void* evicted_values,
                          uint64_t* evicted_scores, uint64_t* evicted_counter,
                          int ignore_evict_strategy);
int hkvo_accum_or_assign(hkvo_table* t, uint64_t n, const uint64_t* keys,
                         const void* value_or_deltas,
                         const uint8_t* accum_or_assigns,
                         const uint64_t* scores, int ignore_evict_strategy);
int hkvo_find_or_insert(hkvo_table* t, uint64_t n, const uint64_t* keys,
                        void* values, const uint64_t* scores,
                        int ignore_evict_strategy);
/* pointer overload: values[i] receives the slot index (not an address) of the
 * row, or UINT64_MAX when the key was refused */
int hkvo_find_or_insert_slot(hkvo_table* t, uint64_t n, const uint64_t* keys,
                             uint64_t* slots, uint8_t* founds,
                             const uint64_t* scores, int ignore_evict_strategy);
int hkvo_assign(hkvo_table* t, uint64_t n, const uint64_t* keys,
                const void* values, const uint64_t* scores);
int hkvo_assign_scores(hkvo_table* t, uint64_t n, const uint64_t* keys,
                       const uint64_t* scores);
int hkvo_assign_values(hkvo_table* t, uint64_t n, const uint64_t* keys,
                       const void* values);
int hkvo_find(const hkvo_table* t, uint64_t n, const uint64_t* keys,
              void* values, uint8_t* founds, uint64_t* scores);
/* find*: slot index of the row or UINT64_MAX */
int hkvo_find_slot(const hkvo_table* t, uint64_t n, const uint64_t* keys,
                   uint64_t* slots, uint8_t* founds, uint64_t* scores);
int hkvo_contains(const hkvo_table* t, uint64_t n, const uint64_t* keys,
                  uint8_t* founds);
/* lock_keys / unlock_keys / find_and_update (merlin_hashtable.cuh:1982-2044,
 * 2811-2843); slot indices stand for the addresses the reference returns */
int hkvo_lock_keys(hkvo_table* t, uint64_t n, const uint64_t* keys, uint64_t* slots,
                   uint8_t* success, const uint64_t* scores);
int hkvo_unlock_keys(hkvo_table* t, uint64_t n, const uint64_t* slots,
                     const uint64_t* keys, uint8_t* success);
int hkvo_find_and_update(hkvo_table* t, uint64_t n, const uint64_t* keys,
                         uint64_t* slots, uint8_t* founds, uint64_t* scores);
int hkvo_erase(hkvo_table* t, uint64_t n, const uint64_t* keys);
/* reserve + rehash (merlin_hashtable.cuh:3503-3541).  Every inserting call
 * above also runs the reference's growth loop first (fast_load_factor >
 * max_load_factor => reserve(2 * capacity), merlin_hashtable.cuh:1151-1154). */
int hkvo_reserve(hkvo_table* t, uint64_t new_capacity);
/* merlin_hashtable.cuh:3561-3579 */
int hkvo_set_max_capacity(hkvo_table* t, uint64_t new_max_capacity);
int hkvo_clear(hkvo_table* t);
int hkvo_export_batch_if(const hkvo_table* t, int predicate, uint64_t pattern,
                         uint64_t threshold, uint64_t n, uint64_t offset,
                         uint64_t* counter, uint64_t* keys, void* values,
                         uint64_t* scores);
uint64_t hkvo_size_if(const hkvo_table* t, int predicate, uint64_t pattern,
                      uint64_t threshold);
uint64_t hkvo_size(const hkvo_table* t);
uint64_t hkvo_capacity(const hkvo_table* t);
uint64_t hkvo_bucket_count(const hkvo_table* t);
/* live keys in one bucket (Table::buckets_size) */
int32_t hkvo_bucket_size(const hkvo_table* t, uint64_t bkt);

/*
 * Multithreaded variants for the reported CPU baseline: the batch is
 * partitioned by bucket, every thread owns a disjoint bucket range and walks
 * its keys in input order, so the table ends up identical to the sequential
 * call.  `threads` <= 0 means one thread per online core.
 */
int hkvo_find_mt(const hkvo_table* t, uint64_t n, const uint64_t* keys,
                 void* values, uint8_t* founds, uint64_t* scores, int threads);
int hkvo_insert_or_assign_mt(hkvo_table* t, uint64_t n, const uint64_t* keys,
                             const void* values, const uint64_t* scores,
                             int ignore_evict_strategy, int threads);
int hkvo_online_cores(void);

#ifdef __cplusplus
}
#endif
#endif
