/*
 * TEST INFRASTRUCTURE ONLY -- see hkv_oracle.h.
 *
 * CPU restatement of the reference's bucketed hash table, written from the
 * text of the reference sources (paths relative to the reference tree):
 *
 *   hash ................ include/merlin/utils.cuh:127-135
 *   digest, addressing .. include/merlin/core_kernels/kernel_utils.cuh:72-103, 626-643
 *   sentinels ........... include/merlin/types.cuh:47-109
 *   score strategies .... include/merlin/core_kernels/kernel_utils.cuh:246-615
 *   upsert per key ...... include/merlin/core_kernels/upsert.cuh:27-234
 *   evicted outputs ..... include/merlin/core_kernels/upsert_and_evict.cuh:151-247
 *   find_or_insert ...... include/merlin/core_kernels/find_or_insert.cuh:149-238
 *   find_or_insert* ..... include/merlin/core_kernels/find_ptr_or_insert.cuh:27-246
 *   accum_or_assign ..... include/merlin/core_kernels/accum_or_assign.cuh:83-174
 *   lookup .............. include/merlin/core_kernels/lookup.cuh:999-1098
 *   lookup (pointer) .... include/merlin/core_kernels/lookup_ptr.cuh:25-152
 *   assign family ....... include/merlin/core_kernels/update.cuh, update_score.cuh,
 *                         update_values.cuh (probe = lookup; score rule =
 *                         ScoreFunctor::update_without_missed)
 *   clear / erase ....... include/merlin/core_kernels.cuh:657-741
 *   export_batch_if ..... include/merlin/core_kernels.cuh:983-1041
 *   bucket count ........ include/merlin/core_kernels.cuh:349-357
 *   argument checks ..... include/merlin_hashtable.cuh:1016-1048, 3832-3861
 *   hybrid refusal rule . include/merlin/core_kernels/upsert.cuh:1524
 *   dual-bucket mode .... include/merlin/core_kernels/dual_bucket_utils.cuh:36-101
 *                         (addressing, digest), dual_bucket_upsert.cuh:139-600
 *                         (insert_or_assign), dual_bucket_lookup.cuh:25-140
 *                         (find: first bucket, then second),
 *                         include/merlin_hashtable.cuh:992-1014 (init checks) and
 *                         the `!is_memory_mode()` guards of the other calls
 *
 * The reference itself cannot be built or run here (CUDA only), and its tests
 * hold no golden vectors (inputs are unseeded).  What pins this file instead
 * (tests/test_oracle_*.py):
 *   - hash: closed-form known answers of fmix64 and the sentinel digests;
 *   - addressing: bucket formula of tests/test_util.cuh:296-331 and the
 *     non-power-of-two bucket count of tests/merlin_hashtable_test.cc.cu:242;
 *   - sentinels: truth table of tests/reserved_keys_test.cc.cu:84-97;
 *   - eviction / refusal: the closed-form scenarios of
 *     tests/merlin_hashtable_test.cc.cu:2674-3053 and an independent brute
 *     force ("a full bucket ends up holding the top-128 scores");
 *   - insert_and_evict: conservation and count identities of
 *     tests/insert_and_evict_test.cc.cu:34-48, 94, 115, 287-311;
 *   - LFU / EpochLFU arithmetic: tests/insert_and_evict_test.cc.cu:541-556,
 *     tests/test_util.cuh:371-376;
 *   - accum_or_assign: tests/accum_or_assign_test.cc.cu:2818-2845;
 *   - export_batch_if / size_if: tests/export_batch_if_test.cc.cu:268-296;
 *   - erase / clear counts: tests/merlin_hashtable_test.cc.cu:336-344;
 *   - dual-bucket mode: closed form of the two bucket indices, the
 *     b1 == b2 case of tests/dual_bucket_test.cc.cu:663-742, first eviction
 *     above load factor 0.98 (:399-465), eviction quality >= 0.995 (:1406-1520),
 *     the guards and init checks (:471-515, 941-1107), clear and re-insert
 *     (:1841-1900).  In this mode a batch is not order-independent (where a
 *     key lands depends on the bucket sizes at that moment); the oracle applies
 *     the batch in input order.
 * Parity unpinned (only an execution of the reference could pin them, and none
 * is observable under the tests' preconditions): victim choice among equal
 * scores, which EMPTY slot an insert takes, and real LRU clock values.
 */
#define _GNU_SOURCE
#include "hkv_oracle.h"

#include <pthread.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>
#include <unistd.h>

#define BUCKET 128u
#define MAX_SCORE UINT64_C(0xFFFFFFFFFFFFFFFF)
#define IGNORED_EPOCH UINT64_C(0xFFFFFFFFFFFFFFFF)
#define EPOCH_MASK UINT64_C(0xFFFFFFFF00000000)
#define LOW32 UINT64_C(0xFFFFFFFF)

struct hkvo_table {
  hkv_options opts;
  int strategy;
  int hybrid_refusal;
  uint64_t buckets_num, capacity;
  uint32_t vb; /* bytes per value row */
  uint64_t empty_key, reclaim_key, locked_key;
  uint64_t rmask1, rmask2, vmask1, vmask2;
  uint8_t empty_digest, reclaim_digest;
  uint8_t* digests;
  uint64_t* keys;
  uint64_t* scores;
  int32_t* sizes;
  uint8_t* values;
  uint64_t epoch;
  int clock_mode;
  uint64_t clock_base;
  int reach_max_capacity; /* merlin_hashtable.cuh:1064 */
  int dual;               /* TableMode::kMemory, merlin_hashtable.cuh:93-98 */
};

static __thread char g_err[512];

const char* hkvo_last_error(void) { return g_err; }

static int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof g_err, fmt, ap);
  va_end(ap);
  return code;
}

/* utils.cuh:127-135 */
uint64_t hkvo_murmur3_fmix64(uint64_t k) {
  k ^= k >> 33;
  k *= UINT64_C(0xff51afd7ed558ccd);
  k ^= k >> 33;
  k *= UINT64_C(0xc4ceb9fe1a85ec53);
  k ^= k >> 33;
  return k;
}

/* types.cuh:47-109 */
int hkvo_reserved_keys(int b, uint64_t out[7]) {
  if (b < 0 || b > 62) return -1;
  if (b == 0) {
    out[0] = UINT64_C(0xFFFFFFFFFFFFFFFF);
    out[1] = UINT64_C(0xFFFFFFFFFFFFFFFE);
    out[2] = UINT64_C(0xFFFFFFFFFFFFFFFD);
    out[3] = out[4] = UINT64_C(0xFFFFFFFFFFFFFFFC);
    out[5] = out[6] = UINT64_C(0xFFFFFFFFFFFFFFFE);
    return 0;
  }
  uint64_t rm1 = ~(UINT64_C(3) << b);
  uint64_t rm2 = rm1 & ~UINT64_C(1);
  uint64_t vm1 = ~(UINT64_C(1) << b);
  uint64_t vm2 = vm1 & ~UINT64_C(1);
  uint64_t empty = rm2 | (UINT64_C(3) << b);
  out[0] = empty;
  out[1] = vm2;
  out[2] = empty & ~(UINT64_C(2) << b);
  out[3] = rm1;
  out[4] = rm2;
  out[5] = vm1;
  out[6] = vm2;
  return 0;
}

/* kernel_utils.cuh:626-643 (modulo, not mask), :84-96 (digest = hash bits 32..39) */
void hkvo_locate(uint64_t key, uint64_t buckets_num, uint64_t* bkt,
                 uint32_t* start, uint8_t* digest) {
  uint64_t h = hkvo_murmur3_fmix64(key);
  uint64_t g = h % (buckets_num * BUCKET);
  *bkt = g / BUCKET;
  uint32_t s = (uint32_t)(g % BUCKET);
  *start = s - (s % 4);
  *digest = (uint8_t)(h >> 32);
}

/* get_dual_bucket_indices, dual_bucket_utils.cuh:36-50; start positions as
 * dual_bucket_upsert.cuh:86-101 (the low and the high hash word, each modulo
 * the capacity, then modulo 128 and rounded down to 4); digest = hash bits
 * 56..63, dual_bucket_utils.cuh:70-74 */
void hkvo_locate_dual(uint64_t key, uint64_t buckets_num, uint64_t bkt[2],
                      uint32_t start[2], uint8_t* digest) {
  uint64_t h = hkvo_murmur3_fmix64(key);
  uint32_t lo = (uint32_t)h, hi = (uint32_t)(h >> 32);
  bkt[0] = lo % buckets_num;
  bkt[1] = hi % buckets_num;
  if (bkt[1] == bkt[0]) bkt[1] = (bkt[1] + 1) % buckets_num;
  uint32_t s0 = (uint32_t)((lo % (buckets_num * BUCKET)) % BUCKET);
  uint32_t s1 = (uint32_t)((hi % (buckets_num * BUCKET)) % BUCKET);
  start[0] = s0 - (s0 % 4);
  start[1] = s1 - (s1 % 4);
  *digest = (uint8_t)(h >> 56);
}

static inline int is_reserved(const hkvo_table* t, uint64_t k) {
  return (k & t->rmask1) == t->rmask2;
}

/* the calls that refuse a dual-bucket table, merlin_hashtable.cuh:1362, 1597,
 * 1705, 1891, 2233, 2304, 2860, 2905, 3505 (MERLIN_CHECK(!is_memory_mode())).
 * The calls the reference leaves unguarded although they probe one bucket
 * only (assign, find*, lock_keys, find_and_update) are refused here as well. */
static int refuse_dual(const hkvo_table* t, const char* what, int guarded) {
  if (!t->dual) return HKV_SUCCESS;
  return fail(guarded ? HKV_ERROR_CHECK : HKV_ERROR_UNSUPPORTED,
              "[MEMORY_MODE] %s is not supported in dual-bucket mode.", what);
}

int hkvo_online_cores(void) {
  long n = sysconf(_SC_NPROCESSORS_ONLN);
  return n < 1 ? 1 : (int)n;
}

/* ---- lifecycle ---------------------------------------------------------- */

static int ispow2_u64(uint64_t x) { return x && !(x & (x - 1)); }

int hkvo_create(const hkv_options* o, int hybrid_refusal, hkvo_table** out) {
  /* merlin_hashtable.cuh:1016-1048 */
  if (o->reserved_key_start_bit < 0 || o->reserved_key_start_bit > 62)
    return fail(HKV_ERROR_CHECK,
                "options.reserved_key_start_bit should >= 0 and <= 62.");
  if (!ispow2_u64(o->max_bucket_size))
    return fail(HKV_ERROR_CHECK, "Bucket size should be the pow of 2");
  if (!ispow2_u64(o->num_of_buckets_per_alloc))
    return fail(HKV_ERROR_CHECK,
                "Then `num_of_buckets_per_alloc` should be the pow of 2");
  if (o->init_capacity < o->num_of_buckets_per_alloc * o->max_bucket_size)
    return fail(HKV_ERROR_CHECK,
                "Then `num_of_buckets_per_alloc` must be equal or less than "
                "initial required buckets number");
  if (o->max_bucket_size != BUCKET)
    return fail(HKV_ERROR_UNSUPPORTED, "only max_bucket_size == 128");
  if (o->io_by_cpu && o->max_hbm_for_vectors != 0)
    return fail(HKV_ERROR_CHECK,
                "`io_by_cpu` should not be true when `max_hbm_for_vectors` is "
                "not 0!");
  if (o->evict_strategy < 0 || o->evict_strategy > 4)
    return fail(HKV_ERROR_ARGUMENT, "bad evict_strategy");
  if (o->dim == 0 || o->value_size == 0)
    return fail(HKV_ERROR_ARGUMENT, "dim and value_size must be positive");

  if (o->table_mode != 0 && o->table_mode != 1)
    return fail(HKV_ERROR_ARGUMENT, "bad table_mode");
  if (o->table_mode == 1) {
    /* merlin_hashtable.cuh:992-1014 */
    if (o->init_capacity != o->max_capacity)
      return fail(HKV_ERROR_CHECK,
                  "[MEMORY_MODE] init_capacity must equal max_capacity. "
                  "Auto-rehash is not supported in dual-bucket mode.");
    if (o->max_hbm_for_vectors != 0)
      return fail(HKV_ERROR_CHECK,
                  "[MEMORY_MODE] Only pure HBM (fast mode) is supported. "
                  "Set max_hbm_for_vectors = 0.");
    if (o->dim * o->value_size > 224 * 4)
      return fail(HKV_ERROR_CHECK,
                  "[MEMORY_MODE] dim * sizeof(V) must not exceed 896 bytes");
    if (o->init_capacity / o->max_bucket_size < 2)
      return fail(HKV_ERROR_CHECK,
                  "[MEMORY_MODE] capacity must provide at least 2 buckets");
  }

  hkvo_table* t = (hkvo_table*)calloc(1, sizeof *t);
  if (!t) return fail(HKV_ERROR_RUNTIME, "out of memory");
  t->opts = *o;
  t->dual = o->table_mode == 1;
  t->strategy = o->evict_strategy;
  t->hybrid_refusal = hybrid_refusal;
  /* core_kernels.cuh:343-357 */
  uint64_t max_size = o->init_capacity > o->max_capacity ? o->init_capacity
                                                         : o->max_capacity;
  if (o->init_capacity * 2 > max_size) {
    t->buckets_num = 1 + (max_size - 1) / BUCKET;
  } else {
    t->buckets_num = 1;
    while (t->buckets_num * BUCKET < o->init_capacity) t->buckets_num *= 2;
  }
  t->capacity = t->buckets_num * BUCKET;
  t->vb = (uint32_t)(o->dim * o->value_size);
  uint64_t rk[7];
  hkvo_reserved_keys(o->reserved_key_start_bit, rk);
  t->empty_key = rk[0];
  t->reclaim_key = rk[1];
  t->locked_key = rk[2];
  t->rmask1 = rk[3];
  t->rmask2 = rk[4];
  t->vmask1 = rk[5];
  t->vmask2 = rk[6];
  t->empty_digest = (uint8_t)(hkvo_murmur3_fmix64(t->empty_key) >> 32);
  t->reclaim_digest = (uint8_t)(hkvo_murmur3_fmix64(t->reclaim_key) >> 32);
  if (t->dual) {
    /* dual_bucket_empty_digest, dual_bucket_utils.cuh:86-90; core_kernels.cuh:67-71 */
    t->empty_digest = (uint8_t)(hkvo_murmur3_fmix64(t->empty_key) >> 56);
    t->reclaim_digest = (uint8_t)(hkvo_murmur3_fmix64(t->reclaim_key) >> 56);
  }
  t->epoch = IGNORED_EPOCH;
  t->reach_max_capacity = t->dual || o->init_capacity * 2 > o->max_capacity;
  t->digests = (uint8_t*)malloc(t->capacity);
  t->keys = (uint64_t*)malloc(t->capacity * 8);
  t->scores = (uint64_t*)calloc(t->capacity, 8);
  t->sizes = (int32_t*)calloc(t->buckets_num, 4);
  t->values = (uint8_t*)calloc(t->capacity, t->vb);
  if (!t->digests || !t->keys || !t->scores || !t->sizes || !t->values) {
    hkvo_destroy(t);
    return fail(HKV_ERROR_RUNTIME, "out of memory");
  }
  /* initialize_buckets, core_kernels.cuh:169-292: key=EMPTY, digest=empty, score=0 */
  memset(t->digests, t->empty_digest, t->capacity);
  for (uint64_t i = 0; i < t->capacity; i++) t->keys[i] = t->empty_key;
  *out = t;
  return HKV_SUCCESS;
}

void hkvo_destroy(hkvo_table* t) {
  if (!t) return;
  free(t->digests);
  free(t->keys);
  free(t->scores);
  free(t->sizes);
  free(t->values);
  free(t);
}

int hkvo_set_global_epoch(hkvo_table* t, uint64_t e) {
  t->epoch = e;
  return HKV_SUCCESS;
}

int hkvo_set_clock(hkvo_table* t, int mode, uint64_t base) {
  t->clock_mode = mode;
  t->clock_base = base;
  return HKV_SUCCESS;
}

uint64_t hkvo_capacity(const hkvo_table* t) { return t->capacity; }
uint64_t hkvo_bucket_count(const hkvo_table* t) { return t->buckets_num; }
int32_t hkvo_bucket_size(const hkvo_table* t, uint64_t b) { return t->sizes[b]; }

uint64_t hkvo_size(const hkvo_table* t) {
  uint64_t s = 0;
  for (uint64_t b = 0; b < t->buckets_num; b++) s += (uint64_t)t->sizes[b];
  return s;
}

/* ---- clock and score strategies ----------------------------------------- */

static inline uint64_t now_ns(const hkvo_table* t, uint64_t i) {
  if (t->clock_mode == 1) return t->clock_base + (i << 20);
  struct timespec ts;
  clock_gettime(CLOCK_REALTIME, &ts); /* %globaltimer counts from the Unix epoch */
  return (uint64_t)ts.tv_sec * UINT64_C(1000000000) + (uint64_t)ts.tv_nsec;
}

static inline void advance_clock(hkvo_table* t) {
  if (t->clock_mode == 1) t->clock_base += UINT64_C(1) << 40;
}

/* check_evict_strategy, merlin_hashtable.cuh:3832-3861 */
static int check_scores_arg(const hkvo_table* t, int strategy,
                            const uint64_t* scores) {
  if ((strategy == HKV_LRU || strategy == HKV_EPOCH_LRU) && scores)
    return fail(HKV_ERROR_CHECK,
                "the scores should not be specified when running on LRU or "
                "Epoch LRU mode.");
  if ((strategy == HKV_LFU || strategy == HKV_EPOCH_LFU) && !scores)
    return fail(HKV_ERROR_CHECK,
                "the scores should be specified when running on LFU or Epoch "
                "LFU mode.");
  if (strategy == HKV_CUSTOMIZED && !scores)
    return fail(HKV_ERROR_CHECK,
                "the scores should be specified when running on customized "
                "mode.");
  if ((strategy == HKV_EPOCH_LRU || strategy == HKV_EPOCH_LFU) &&
      t->epoch == IGNORED_EPOCH)
    return fail(HKV_ERROR_CHECK,
                "the global_epoch is invalid and should be assigned by calling "
                "`set_global_epoch` when running on Epoch LRU or Epoch LFU "
                "mode.");
  return HKV_SUCCESS;
}

/* ScoreFunctor<Strategy>::desired_when_missed, kernel_utils.cuh:275-279,
 * 332-336, 403-411, 464-471, 567-571 */
static inline uint64_t desired_when_missed(const hkvo_table* t, int strategy,
                                           const uint64_t* in, uint64_t i) {
  switch (strategy) {
    case HKV_LRU:
      return now_ns(t, i);
    case HKV_LFU:
      return MAX_SCORE;
    case HKV_EPOCH_LRU:
      if (t->epoch == IGNORED_EPOCH && in) return in[i];
      return (t->epoch << 32) | ((now_ns(t, i) >> 20) & LOW32);
    case HKV_EPOCH_LFU:
      if (t->epoch == IGNORED_EPOCH) return in[i];
      return (t->epoch << 32) | (in[i] & LOW32);
    default:
      return in[i];
  }
}

/* ScoreFunctor<Strategy>::update_with_digest, kernel_utils.cuh:291-302,
 * 353-371, 422-434, 490-517, 581-593.  Returns 0 when the functor writes
 * nothing (LFU without input scores). */
static inline int score_on_upsert(const hkvo_table* t, int strategy,
                                  const uint64_t* in, uint64_t i,
                                  uint64_t desired, int new_insert,
                                  uint64_t old, uint64_t* out) {
  switch (strategy) {
    case HKV_LRU:
      *out = now_ns(t, i);
      return 1;
    case HKV_LFU:
      if (!in) return 0;
      *out = new_insert ? in[i] : in[i] + old;
      return 1;
    case HKV_EPOCH_LFU: {
      uint64_t s = desired;
      if (!new_insert) {
        s = old & LOW32;
        if (LOW32 - s > (desired & LOW32))
          s += desired;
        else
          s = (desired & EPOCH_MASK) | LOW32;
      }
      *out = s;
      return 1;
    }
    default: /* EpochLRU, Customized */
      *out = desired;
      return 1;
  }
}

/* ScoreFunctor<Strategy>::update_without_missed, kernel_utils.cuh:304-321,
 * 373-392, 436-453, 519-557, 594-612 (assign family) */
static inline int score_on_assign(const hkvo_table* t, const uint64_t* in,
                                  uint64_t i, uint64_t old, uint64_t* out) {
  switch (t->strategy) {
    case HKV_LRU:
      *out = now_ns(t, i);
      return 1;
    case HKV_LFU:
      if (!in) return 0;
      *out = old + in[i];
      return 1;
    case HKV_EPOCH_LRU:
      *out = (t->epoch << 32) | ((now_ns(t, i) >> 20) & LOW32);
      return 1;
    case HKV_EPOCH_LFU: {
      if (!in) return 0;
      uint64_t s = old & LOW32;
      if (LOW32 - s > (in[i] & LOW32))
        s += (t->epoch << 32) | (in[i] & LOW32);
      else
        s = (t->epoch << 32) | LOW32;
      *out = s;
      return 1;
    }
    default:
      if (!in) return 0;
      *out = in[i];
      return 1;
  }
}

/* ---- probing ------------------------------------------------------------- */

/* exact-match lookup in the key's bucket; returns slot index or -1 */
static inline int64_t lookup_slot(const hkvo_table* t, uint64_t key) {
  uint64_t bkt;
  uint32_t start;
  uint8_t dg;
  if (t->dual) {
    /* dual_bucket_lookup.cuh:25-140: the first bucket, then the second */
    uint64_t b[2];
    uint32_t st[2];
    hkvo_locate_dual(key, t->buckets_num, b, st, &dg);
    for (int w = 0; w < 2; w++) {
      const uint8_t* d = t->digests + b[w] * BUCKET;
      const uint64_t* k = t->keys + b[w] * BUCKET;
      for (uint32_t p = 0; p < BUCKET; p++)
        if (d[p] == dg && k[p] == key) return (int64_t)(b[w] * BUCKET + p);
    }
    return -1;
  }
  hkvo_locate(key, t->buckets_num, &bkt, &start, &dg);
  const uint8_t* d = t->digests + bkt * BUCKET;
  const uint64_t* k = t->keys + bkt * BUCKET;
  for (uint32_t p = 0; p < BUCKET; p++)
    if (d[p] == dg && k[p] == key) return (int64_t)(bkt * BUCKET + p);
  return -1;
}

typedef enum {
  OCC_DUPLICATE,
  OCC_EMPTY,
  OCC_RECLAIMED,
  OCC_EVICT,
  OCC_REFUSED
} occ_t;

typedef struct {
  occ_t result;
  uint64_t bkt;
  uint32_t pos;
  uint8_t digest;
  uint64_t desired;   /* score the key would get when missed */
  uint64_t min_score; /* scanned minimum (evict / refuse) */
  uint64_t victim;    /* key found in the victim slot */
} occupy_t;

/*
 * Decide what an upsert-family operation does with `key`; the table is not
 * modified.  Follows upsert.cuh:52-223:
 *   1. digest-matching slots, in 16-byte chunks from align16(start), wrapping;
 *   2. the first EMPTY slot in the same order (slots below `start` in the
 *      first chunk are skipped and seen again by the extra last chunk), only
 *      when the bucket is not full;
 *   3. minimum over all 128 score slots, strict '<' so the lowest index wins
 *      ties; refuse when desired < min.  With `ptr_rule` (the lock-key kernels
 *      of the pointer overload and of hybrid mode, find_ptr_or_insert.cuh:
 *      170-200, upsert.cuh:1478-1524) slots whose key is LOCKED or EMPTY are
 *      skipped by the scan and the refusal test is desired <= min.
 */
static void decide(const hkvo_table* t, int strategy, uint64_t key,
                   const uint64_t* in_scores, uint64_t i, int ptr_rule,
                   occupy_t* r) {
  uint32_t start;
  hkvo_locate(key, t->buckets_num, &r->bkt, &start, &r->digest);
  r->desired = desired_when_missed(t, strategy, in_scores, i);
  const uint8_t* d = t->digests + r->bkt * BUCKET;
  const uint64_t* k = t->keys + r->bkt * BUCKET;
  const uint64_t* s = t->scores + r->bkt * BUCKET;
  const int full = t->sizes[r->bkt] == (int32_t)BUCKET;
  /* The reference meets the key before any EMPTY slot when it probes from the start
   * position, because its rehash compacts a bucket after moving keys out of it
   * (defragmentation_for_rehash, core_kernels.cuh:445-492).  The rehash here leaves
   * the holes where they are, so the key is looked for in the whole bucket first. */
  for (uint32_t p = 0; p < BUCKET; p++) {
    if (d[p] == r->digest && k[p] == key) {
      r->result = OCC_DUPLICATE;
      r->pos = p;
      return;
    }
  }
  uint32_t base = start & ~15u;
  for (uint32_t off = 0; !full && off < BUCKET + 16; off += 16) {
    uint32_t cur = (base + off) & (BUCKET - 1);
    for (uint32_t w = 0; w < 4; w++) {
      for (uint32_t b = 0; b < 4; b++) {
        uint32_t p = cur + w * 4 + b;
        if (d[p] != t->empty_digest) continue;
        if (off == 0 && p < start) continue;
        if (k[p] == t->empty_key) {
          r->result = OCC_EMPTY;
          r->pos = p;
          return;
        }
      }
    }
  }
  uint64_t min_score = MAX_SCORE;
  int min_pos = -1;
  for (uint32_t p = 0; p < BUCKET; p++) {
    if (s[p] < min_score) {
      /* a slot that lock_keys holds is never a victim: the reference's plain
       * kernels would retry such a slot for ever (upsert.cuh:192-222) */
      if (k[p] == t->locked_key) continue;
      if (ptr_rule && k[p] == t->empty_key) continue;
      min_score = s[p];
      min_pos = (int)p;
    }
  }
  r->min_score = min_score;
  int refuse = ptr_rule ? (r->desired <= min_score) : (r->desired < min_score);
  if (refuse || min_pos < 0) {
    r->result = OCC_REFUSED;
    return;
  }
  r->pos = (uint32_t)min_pos;
  r->victim = k[min_pos];
  r->result = (r->victim == t->reclaim_key) ? OCC_RECLAIMED : OCC_EVICT;
}

/*
 * The same decision in dual-bucket mode, dual_bucket_upsert.cuh:139-600:
 *   0. the key is looked for in both buckets (first b1, then b2);
 *   1. otherwise the bucket with fewer keys is tried first (b1 on a tie), then
 *      the other: in a bucket that is not full the first EMPTY slot in
 *      circular order from the bucket's own start position is taken;
 *   2. otherwise the minimum score over both buckets decides: refuse when
 *      desired < min; the victim is the minimum of b1 when min1 <= min2, else
 *      of b2 (lowest slot on ties; the reference's choice among equal scores
 *      depends on its lane layout and is not reproduced).
 */
static void decide_dual(const hkvo_table* t, int strategy, uint64_t key,
                        const uint64_t* in_scores, uint64_t i, occupy_t* r) {
  uint64_t b[2];
  uint32_t st[2];
  hkvo_locate_dual(key, t->buckets_num, b, st, &r->digest);
  r->desired = desired_when_missed(t, strategy, in_scores, i);
  for (int w = 0; w < 2; w++) {
    const uint8_t* d = t->digests + b[w] * BUCKET;
    const uint64_t* k = t->keys + b[w] * BUCKET;
    for (uint32_t p = 0; p < BUCKET; p++)
      if (d[p] == r->digest && k[p] == key) {
        r->result = OCC_DUPLICATE;
        r->bkt = b[w];
        r->pos = p;
        return;
      }
  }
  const int first = t->sizes[b[0]] <= t->sizes[b[1]] ? 0 : 1;
  for (int turn = 0; turn < 2; turn++) {
    const int w = turn == 0 ? first : 1 - first;
    if (t->sizes[b[w]] >= (int32_t)BUCKET) continue;
    const uint8_t* d = t->digests + b[w] * BUCKET;
    const uint64_t* k = t->keys + b[w] * BUCKET;
    for (uint32_t off = 0; off < BUCKET; off++) {
      uint32_t p = (st[w] + off) & (BUCKET - 1);
      if (d[p] == t->empty_digest && k[p] == t->empty_key) {
        r->result = OCC_EMPTY;
        r->bkt = b[w];
        r->pos = p;
        return;
      }
    }
  }
  uint64_t mins[2] = {MAX_SCORE, MAX_SCORE};
  int pos[2] = {-1, -1};
  for (int w = 0; w < 2; w++) {
    const uint64_t* k = t->keys + b[w] * BUCKET;
    const uint64_t* s = t->scores + b[w] * BUCKET;
    for (uint32_t p = 0; p < BUCKET; p++) {
      if (k[p] == t->locked_key || k[p] == t->empty_key) continue;
      if (s[p] < mins[w]) {
        mins[w] = s[p];
        pos[w] = (int)p;
      }
    }
  }
  const int w = mins[0] <= mins[1] ? 0 : 1;
  r->min_score = mins[w];
  if (r->desired < mins[w] || pos[w] < 0) {
    r->result = OCC_REFUSED;
    return;
  }
  r->bkt = b[w];
  r->pos = (uint32_t)pos[w];
  r->victim = t->keys[b[w] * BUCKET + (uint32_t)pos[w]];
  r->result = (r->victim == t->reclaim_key) ? OCC_RECLAIMED : OCC_EVICT;
}

/* digest + score + bucket size for an accepted key (update_with_digest and
 * the atomicAdd on buckets_size, upsert.cuh:112-146, 203-215) */
static void commit_meta(hkvo_table* t, int strategy, const occupy_t* r,
                        const uint64_t* in_scores, uint64_t i) {
  uint64_t slot = r->bkt * BUCKET + r->pos;
  uint64_t ns;
  int new_insert = r->result != OCC_DUPLICATE;
  if (score_on_upsert(t, strategy, in_scores, i, r->desired, new_insert,
                      t->scores[slot], &ns)) {
    t->digests[slot] = r->digest;
    t->scores[slot] = ns;
  }
  if (r->result == OCC_EMPTY || r->result == OCC_RECLAIMED) t->sizes[r->bkt]++;
}

/* ---- growth -------------------------------------------------------------------
 * reserve (merlin_hashtable.cuh:3503-3541): while capacity < new_capacity and
 * doubling stays within max_capacity, double the number of buckets
 * (double_capacity, core_kernels.cuh:386-401) and move every live key whose
 * bucket changed (rehash_kernel_for_fast_mode, core_kernels.cuh:540-591; the
 * key goes to the first EMPTY slot of its new bucket at or after its start
 * position, move_key_to_new_bucket :494-537).  Tombstones stay where they are.
 * The reference also compacts the old bucket towards start positions
 * (defragmentation_for_rehash :445-492); slot positions are not observable
 * through the API and lookups here scan the whole bucket, so that step is left
 * out. */
static int double_capacity(hkvo_table* t) {
  const uint64_t ob = t->buckets_num, nb = ob * 2, ncap = nb * BUCKET;
  uint8_t* dg = (uint8_t*)realloc(t->digests, ncap);
  if (dg) t->digests = dg;
  uint64_t* ks = (uint64_t*)realloc(t->keys, ncap * 8);
  if (ks) t->keys = ks;
  uint64_t* sc = (uint64_t*)realloc(t->scores, ncap * 8);
  if (sc) t->scores = sc;
  int32_t* sz = (int32_t*)realloc(t->sizes, nb * 4);
  if (sz) t->sizes = sz;
  uint8_t* vs = (uint8_t*)realloc(t->values, ncap * (uint64_t)t->vb);
  if (vs) t->values = vs;
  if (!dg || !ks || !sc || !sz || !vs) return fail(HKV_ERROR_RUNTIME, "out of memory");
  memset(t->digests + t->capacity, t->empty_digest, ncap - t->capacity);
  for (uint64_t i = t->capacity; i < ncap; i++) t->keys[i] = t->empty_key;
  memset(t->scores + t->capacity, 0, (ncap - t->capacity) * 8);
  memset(t->sizes + ob, 0, ob * 4);
  memset(t->values + t->capacity * (uint64_t)t->vb, 0, (ncap - t->capacity) * (uint64_t)t->vb);
  t->buckets_num = nb;
  t->capacity = ncap;
  for (uint64_t b = 0; b < ob; b++) {
    for (uint64_t p = 0; p < BUCKET; p++) {
      const uint64_t s = b * BUCKET + p;
      const uint64_t k = t->keys[s];
      if (k == t->empty_key || k == t->reclaim_key) continue;
      uint64_t nbkt;
      uint32_t start;
      uint8_t digest;
      hkvo_locate(k, nb, &nbkt, &start, &digest);
      if (nbkt == b) continue;
      uint64_t d = UINT64_MAX;
      for (uint64_t off = 0; off < BUCKET; off++) {
        const uint64_t q = nbkt * BUCKET + ((start + off) & (BUCKET - 1));
        if (t->keys[q] == t->empty_key) {
          d = q;
          break;
        }
      }
      if (d == UINT64_MAX) return fail(HKV_ERROR_RUNTIME, "rehash: new bucket is full");
      t->keys[d] = k;
      t->digests[d] = t->digests[s];
      t->scores[d] = t->scores[s];
      memcpy(t->values + d * t->vb, t->values + s * t->vb, t->vb);
      t->sizes[nbkt]++;
      t->keys[s] = t->empty_key;
      t->digests[s] = t->empty_digest;
      t->sizes[b]--;
    }
  }
  return HKV_SUCCESS;
}

int hkvo_reserve(hkvo_table* t, uint64_t new_capacity) {
  {
    int drc = refuse_dual(t, "reserve()", 1);
    if (drc) return drc;
  }
  if (t->reach_max_capacity || new_capacity > t->opts.max_capacity) {
    t->reach_max_capacity = t->capacity * 2 > t->opts.max_capacity;
    return HKV_SUCCESS;
  }
  while (t->capacity < new_capacity && t->capacity * 2 <= t->opts.max_capacity) {
    int rc = double_capacity(t);
    if (rc) return rc;
  }
  t->reach_max_capacity = t->capacity * 2 > t->opts.max_capacity;
  return HKV_SUCCESS;
}

/* set_max_capacity, merlin_hashtable.cuh:3561-3579 */
int hkvo_set_max_capacity(hkvo_table* t, uint64_t new_max_capacity) {
  if (!ispow2_u64(new_max_capacity))
    return fail(HKV_ERROR_ARGUMENT, "None power-of-2 new_max_capacity is not supported.");
  if (new_max_capacity < t->capacity) return HKV_SUCCESS;
  t->reach_max_capacity = 0;
  t->opts.max_capacity = new_max_capacity;
  return HKV_SUCCESS;
}

/* fast_load_factor, merlin_hashtable.cuh:3796-3830: sizes of the first
 * min(buckets, 1024) buckets, plus the incoming batch as if it were all new */
static float fast_load_factor(const hkvo_table* t, uint64_t delta) {
  const uint64_t N = t->buckets_num < 1024 ? t->buckets_num : 1024;
  int64_t sum = 0;
  for (uint64_t b = 0; b < N; b++) sum += t->sizes[b];
  return (float)((delta * 1.0) / (t->capacity * 1.0) + (sum * 1.0) / (BUCKET * N * 1.0));
}

/* the growth loop at the head of every inserting call
 * (merlin_hashtable.cuh:1151-1154, 1369-1372, 1604-1607, 1712-1715, 1898-1901) */
static int grow_for(hkvo_table* t, uint64_t n) {
  while (!t->reach_max_capacity && fast_load_factor(t, n) > t->opts.max_load_factor) {
    int rc = hkvo_reserve(t, t->capacity * 2);
    if (rc) return rc;
  }
  return HKV_SUCCESS;
}

static inline int strategy_of(const hkvo_table* t, int ignore) {
  return ignore ? HKV_CUSTOMIZED : t->strategy;
}

/* ---- upsert family --------------------------------------------------------- */

static void upsert_one(hkvo_table* t, int strategy, uint64_t i,
                       const uint64_t* keys, const uint8_t* values,
                       const uint64_t* scores) {
  uint64_t key = keys[i];
  if (is_reserved(t, key)) return;
  occupy_t r;
  if (t->dual)
    decide_dual(t, strategy, key, scores, i, &r);
  else
    decide(t, strategy, key, scores, i, 0, &r);
  if (r.result == OCC_REFUSED) return;
  commit_meta(t, strategy, &r, scores, i);
  uint64_t slot = r.bkt * BUCKET + r.pos;
  memcpy(t->values + slot * t->vb, values + i * t->vb, t->vb);
  t->keys[slot] = key;
}


/*
 * Hybrid mode (values partly in host memory) runs two kernels per call
 * (upsert.cuh:1350-1595, find_or_insert.cuh:1417-1676): the first locks one
 * slot per key -- the key word stays LOCKED, digest and score are already
 * final -- and the second moves the value rows and stores the keys.  Slots
 * taken earlier in the same batch are therefore invisible to the victim scan
 * of later keys.  `dup_reads` selects find_or_insert's direction for hits.
 */
static int upsert_two_phase(hkvo_table* t, int strategy, uint64_t n,
                            const uint64_t* keys, uint8_t* values,
                            const uint64_t* scores, int dup_reads) {
  uint64_t* slot_of = (uint64_t*)malloc(n * 8);
  uint8_t* dup = (uint8_t*)malloc(n);
  if (!slot_of || !dup) {
    free(slot_of);
    free(dup);
    return fail(HKV_ERROR_RUNTIME, "out of memory");
  }
  for (uint64_t i = 0; i < n; i++) {
    slot_of[i] = UINT64_MAX;
    uint64_t key = keys[i];
    if (is_reserved(t, key)) continue;
    occupy_t r;
    decide(t, strategy, key, scores, i, 1, &r);
    if (r.result == OCC_REFUSED) continue;
    commit_meta(t, strategy, &r, scores, i);
    slot_of[i] = r.bkt * BUCKET + r.pos;
    dup[i] = r.result == OCC_DUPLICATE;
    t->keys[slot_of[i]] = t->locked_key;
  }
  for (uint64_t i = 0; i < n; i++) {
    uint64_t slot = slot_of[i];
    if (slot == UINT64_MAX) continue;
    if (dup_reads && dup[i])
      memcpy(values + i * t->vb, t->values + slot * t->vb, t->vb);
    else
      memcpy(t->values + slot * t->vb, values + i * t->vb, t->vb);
    t->keys[slot] = keys[i];
  }
  free(slot_of);
  free(dup);
  return HKV_SUCCESS;
}

int hkvo_insert_or_assign(hkvo_table* t, uint64_t n, const uint64_t* keys,
                          const void* values, const uint64_t* scores,
                          int ignore) {
  if (n == 0) return HKV_SUCCESS;
  {
    int grc = grow_for(t, n);
    if (grc) return grc;
  }
  int strategy = strategy_of(t, ignore);
  if (!ignore) {
    int rc = check_scores_arg(t, strategy, scores);
    if (rc) return rc;
  }
  if (t->hybrid_refusal) {
    int rc = upsert_two_phase(t, strategy, n, keys, (uint8_t*)values, scores, 0);
    if (rc) return rc;
  } else {
    for (uint64_t i = 0; i < n; i++)
      upsert_one(t, strategy, i, keys, (const uint8_t*)values, scores);
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

int hkvo_insert_and_evict(hkvo_table* t, uint64_t n, const uint64_t* keys,
                          const void* values_, const uint64_t* scores,
                          uint64_t* ek, void* ev_, uint64_t* es,
                          uint64_t* counter, int ignore) {
  {
    int drc = refuse_dual(t, "insert_and_evict()", 1);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  {
    int grc = grow_for(t, n);
    if (grc) return grc;
  }
  if (t->hybrid_refusal) /* merlin_hashtable.cuh:1384-1386 */
    return fail(HKV_ERROR_RUNTIME,
                "insert_and_evict is not supported in hybrid mode");
  int strategy = strategy_of(t, ignore);
  if (!ignore) {
    int rc = check_scores_arg(t, strategy, scores);
    if (rc) return rc;
  }
  const uint8_t* values = (const uint8_t*)values_;
  uint8_t* ev = (uint8_t*)ev_;
  for (uint64_t i = 0; i < n; i++) {
    uint64_t key = keys[i];
    if (is_reserved(t, key)) continue;
    occupy_t r;
    decide(t, strategy, key, scores, i, 0, &r);
    if (r.result == OCC_REFUSED) { /* upsert_and_evict.cuh:188-194, 243-245 */
      uint64_t idx = (*counter)++;
      ek[idx] = key;
      if (es) es[idx] = r.desired;
      memcpy(ev + idx * t->vb, values + i * t->vb, t->vb);
      continue;
    }
    uint64_t slot = r.bkt * BUCKET + r.pos;
    if (r.result == OCC_EVICT) { /* :218-224, 236-238 */
      uint64_t idx = (*counter)++;
      ek[idx] = r.victim;
      if (es) es[idx] = r.min_score;
      memcpy(ev + idx * t->vb, t->values + slot * t->vb, t->vb);
    }
    commit_meta(t, strategy, &r, scores, i);
    memcpy(t->values + slot * t->vb, values + i * t->vb, t->vb);
    t->keys[slot] = key;
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

int hkvo_find_or_insert(hkvo_table* t, uint64_t n, const uint64_t* keys,
                        void* values_, const uint64_t* scores, int ignore) {
  {
    int drc = refuse_dual(t, "find_or_insert()", 1);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  {
    int grc = grow_for(t, n);
    if (grc) return grc;
  }
  int strategy = strategy_of(t, ignore);
  if (!ignore) {
    int rc = check_scores_arg(t, strategy, scores);
    if (rc) return rc;
  }
  uint8_t* values = (uint8_t*)values_;
  if (t->hybrid_refusal) {
    int rc = upsert_two_phase(t, strategy, n, keys, values, scores, 1);
    if (rc) return rc;
    advance_clock(t);
    return HKV_SUCCESS;
  }
  for (uint64_t i = 0; i < n; i++) {
    uint64_t key = keys[i];
    if (is_reserved(t, key)) continue;
    occupy_t r;
    decide(t, strategy, key, scores, i, 0, &r);
    if (r.result == OCC_REFUSED) continue;
    commit_meta(t, strategy, &r, scores, i);
    uint64_t slot = r.bkt * BUCKET + r.pos;
    if (r.result == OCC_DUPLICATE) /* find_or_insert.cuh:227-232 */
      memcpy(values + i * t->vb, t->values + slot * t->vb, t->vb);
    else
      memcpy(t->values + slot * t->vb, values + i * t->vb, t->vb);
    t->keys[slot] = key;
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

int hkvo_find_or_insert_slot(hkvo_table* t, uint64_t n, const uint64_t* keys,
                             uint64_t* slots, uint8_t* founds,
                             const uint64_t* scores, int ignore) {
  {
    int drc = refuse_dual(t, "find_or_insert()", 1);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  {
    int grc = grow_for(t, n);
    if (grc) return grc;
  }
  int strategy = strategy_of(t, ignore);
  if (!ignore) {
    int rc = check_scores_arg(t, strategy, scores);
    if (rc) return rc;
  }
  for (uint64_t i = 0; i < n; i++) {
    uint64_t key = keys[i];
    if (is_reserved(t, key)) continue; /* outputs untouched, :66-68 */
    occupy_t r;
    decide(t, strategy, key, scores, i, 1, &r);
    founds[i] = r.result == OCC_DUPLICATE;
    if (r.result == OCC_REFUSED) {
      slots[i] = UINT64_MAX;
      continue;
    }
    commit_meta(t, strategy, &r, scores, i);
    uint64_t slot = r.bkt * BUCKET + r.pos;
    slots[i] = slot;
    t->keys[slot] = key;
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

static void add_row(int kind, uint8_t* dst, const uint8_t* delta, uint64_t dim) {
  switch (kind) {
    case HKV_VALUE_F32: {
      float* d = (float*)dst;
      const float* s = (const float*)delta;
      for (uint64_t j = 0; j < dim; j++) d[j] += s[j];
      break;
    }
    case HKV_VALUE_F64: {
      double* d = (double*)dst;
      const double* s = (const double*)delta;
      for (uint64_t j = 0; j < dim; j++) d[j] += s[j];
      break;
    }
    case HKV_VALUE_I32: {
      uint32_t* d = (uint32_t*)dst;
      const uint32_t* s = (const uint32_t*)delta;
      for (uint64_t j = 0; j < dim; j++) d[j] += s[j];
      break;
    }
    case HKV_VALUE_I64: {
      uint64_t* d = (uint64_t*)dst;
      const uint64_t* s = (const uint64_t*)delta;
      for (uint64_t j = 0; j < dim; j++) d[j] += s[j];
      break;
    }
    case HKV_VALUE_I8: {
      for (uint64_t j = 0; j < dim; j++) dst[j] = (uint8_t)(dst[j] + delta[j]);
      break;
    }
    case HKV_VALUE_I16: {
      uint16_t* d = (uint16_t*)dst;
      const uint16_t* s = (const uint16_t*)delta;
      for (uint64_t j = 0; j < dim; j++) d[j] = (uint16_t)(d[j] + s[j]);
      break;
    }
    default:
      break;
  }
}

int hkvo_accum_or_assign(hkvo_table* t, uint64_t n, const uint64_t* keys,
                         const void* vd_, const uint8_t* flags,
                         const uint64_t* scores, int ignore) {
  {
    int drc = refuse_dual(t, "accum_or_assign()", 1);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  {
    int grc = grow_for(t, n);
    if (grc) return grc;
  }
  if (t->opts.value_kind == HKV_VALUE_BYTES)
    return fail(HKV_ERROR_ARGUMENT, "accum_or_assign needs an arithmetic value_kind");
  int strategy = strategy_of(t, ignore);
  if (!ignore) {
    int rc = check_scores_arg(t, strategy, scores);
    if (rc) return rc;
  }
  const uint8_t* vd = (const uint8_t*)vd_;
  for (uint64_t i = 0; i < n; i++) {
    uint64_t key = keys[i];
    if (is_reserved(t, key)) continue;
    occupy_t r;
    decide(t, strategy, key, scores, i, 0, &r);
    if (r.result == OCC_REFUSED) continue;
    int is_accum = flags[i] != 0;
    int dup = r.result == OCC_DUPLICATE;
    if (is_accum != dup) continue; /* slot restored, accum_or_assign.cuh:139-156 */
    commit_meta(t, strategy, &r, scores, i);
    uint64_t slot = r.bkt * BUCKET + r.pos;
    if (is_accum)
      add_row(t->opts.value_kind, t->values + slot * t->vb, vd + i * t->vb,
              t->opts.dim);
    else
      memcpy(t->values + slot * t->vb, vd + i * t->vb, t->vb);
    t->keys[slot] = key;
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

/* ---- assign family --------------------------------------------------------- */

static int assign_impl(hkvo_table* t, uint64_t n, const uint64_t* keys,
                       const uint8_t* values, const uint64_t* scores,
                       int touch_scores) {
  for (uint64_t i = 0; i < n; i++) {
    uint64_t key = keys[i];
    if (is_reserved(t, key)) continue;
    int64_t slot = lookup_slot(t, key);
    if (slot < 0) continue;
    if (touch_scores) {
      uint64_t ns;
      if (score_on_assign(t, scores, i, t->scores[slot], &ns)) t->scores[slot] = ns;
    }
    if (values) memcpy(t->values + (uint64_t)slot * t->vb, values + i * t->vb, t->vb);
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

int hkvo_assign(hkvo_table* t, uint64_t n, const uint64_t* keys,
                const void* values, const uint64_t* scores) {
  {
    int drc = refuse_dual(t, "assign()", 0);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  int rc = check_scores_arg(t, t->strategy, scores);
  if (rc) return rc;
  return assign_impl(t, n, keys, (const uint8_t*)values, scores, 1);
}

int hkvo_assign_scores(hkvo_table* t, uint64_t n, const uint64_t* keys,
                       const uint64_t* scores) {
  {
    int drc = refuse_dual(t, "assign_scores()", 1);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  int rc = check_scores_arg(t, t->strategy, scores);
  if (rc) return rc;
  return assign_impl(t, n, keys, NULL, scores, 1);
}

int hkvo_assign_values(hkvo_table* t, uint64_t n, const uint64_t* keys,
                       const void* values) {
  {
    int drc = refuse_dual(t, "assign_values()", 1);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  return assign_impl(t, n, keys, (const uint8_t*)values, NULL, 0);
}

/* ---- read-only ops --------------------------------------------------------- */

static inline void find_one(const hkvo_table* t, uint64_t i, const uint64_t* keys,
                            uint8_t* values, uint8_t* founds, uint64_t* scores) {
  uint64_t key = keys[i];
  founds[i] = 0;
  if (is_reserved(t, key)) return;
  int64_t slot = lookup_slot(t, key);
  if (slot < 0) return;
  founds[i] = 1;
  if (values) memcpy(values + i * t->vb, t->values + (uint64_t)slot * t->vb, t->vb);
  if (scores) scores[i] = t->scores[slot];
}

int hkvo_find(const hkvo_table* t, uint64_t n, const uint64_t* keys,
              void* values, uint8_t* founds, uint64_t* scores) {
  for (uint64_t i = 0; i < n; i++)
    find_one(t, i, keys, (uint8_t*)values, founds, scores);
  return HKV_SUCCESS;
}

int hkvo_find_slot(const hkvo_table* t, uint64_t n, const uint64_t* keys,
                   uint64_t* slots, uint8_t* founds, uint64_t* scores) {
  {
    int drc = refuse_dual(t, "find() by pointer", 0);
    if (drc) return drc;
  }
  for (uint64_t i = 0; i < n; i++) {
    int64_t slot = is_reserved(t, keys[i]) ? -1 : lookup_slot(t, keys[i]);
    founds[i] = slot >= 0;
    slots[i] = slot >= 0 ? (uint64_t)slot : UINT64_MAX;
    if (slot >= 0 && scores) scores[i] = t->scores[slot];
  }
  return HKV_SUCCESS;
}

/* score of a key that is present, as the upsert kernels leave it
 * (update_with_digest with is_insert = false) */
static void touch_score(hkvo_table* t, uint64_t slot, const uint64_t* in, uint64_t i) {
  uint64_t ns;
  const uint64_t desired = desired_when_missed(t, t->strategy, in, i);
  if (score_on_upsert(t, t->strategy, in, i, desired, 0, t->scores[slot], &ns))
    t->scores[slot] = ns;
}

/* lock_keys (merlin_hashtable.cuh:1982-2012, lock_kernel_with_filter,
 * core_kernels.cuh:1248-1362): a key that is present has its key word replaced
 * by LOCKED and its score touched; slots[i] = its slot (the reference returns
 * the address of the key word) or UINT64_MAX.  The score argument is checked
 * as in the other calls; the reference does not check it here and reads
 * through a null pointer when a strategy needs scores that were not given. */
int hkvo_lock_keys(hkvo_table* t, uint64_t n, const uint64_t* keys, uint64_t* slots,
                   uint8_t* success, const uint64_t* scores) {
  {
    int drc = refuse_dual(t, "lock_keys()", 0);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  int rc = check_scores_arg(t, t->strategy, scores);
  if (rc) return rc;
  for (uint64_t i = 0; i < n; i++) {
    int64_t slot = is_reserved(t, keys[i]) ? -1 : lookup_slot(t, keys[i]);
    slots[i] = slot >= 0 ? (uint64_t)slot : UINT64_MAX;
    if (success) success[i] = slot >= 0;
    if (slot < 0) continue;
    t->keys[slot] = t->locked_key;
    touch_score(t, (uint64_t)slot, scores, i);
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

/* unlock_keys (merlin_hashtable.cuh:2026-2044, unlock_keys_kernel,
 * core_kernels.cuh:1180-1204) */
int hkvo_unlock_keys(hkvo_table* t, uint64_t n, const uint64_t* slots,
                     const uint64_t* keys, uint8_t* success) {
  {
    int drc = refuse_dual(t, "unlock_keys()", 0);
    if (drc) return drc;
  }
  for (uint64_t i = 0; i < n; i++) {
    int ok = slots[i] != UINT64_MAX && t->keys[slots[i]] == t->locked_key;
    if (ok) t->keys[slots[i]] = keys[i];
    if (success) success[i] = (uint8_t)ok;
  }
  return HKV_SUCCESS;
}

/* find_and_update (merlin_hashtable.cuh:2811-2843,
 * tlp_lookup_ptr_kernel_with_filter with update_score = true,
 * lookup_ptr.cuh:25-150): find* that also touches the score of every key it
 * finds; scores[i] returns the score after the touch. */
int hkvo_find_and_update(hkvo_table* t, uint64_t n, const uint64_t* keys,
                         uint64_t* slots, uint8_t* founds, uint64_t* scores) {
  {
    int drc = refuse_dual(t, "find_and_update()", 0);
    if (drc) return drc;
  }
  if (n == 0) return HKV_SUCCESS;
  int rc = check_scores_arg(t, t->strategy, scores);
  if (rc) return rc;
  for (uint64_t i = 0; i < n; i++) {
    int64_t slot = is_reserved(t, keys[i]) ? -1 : lookup_slot(t, keys[i]);
    if (founds) founds[i] = slot >= 0;
    slots[i] = slot >= 0 ? (uint64_t)slot : UINT64_MAX;
    if (slot < 0) continue;
    touch_score(t, (uint64_t)slot, scores, i);
    if (scores) scores[i] = t->scores[slot];
  }
  advance_clock(t);
  return HKV_SUCCESS;
}

int hkvo_contains(const hkvo_table* t, uint64_t n, const uint64_t* keys,
                  uint8_t* founds) {
  {
    int drc = refuse_dual(t, "contains()", 1);
    if (drc) return drc;
  }
  for (uint64_t i = 0; i < n; i++)
    founds[i] = !is_reserved(t, keys[i]) && lookup_slot(t, keys[i]) >= 0;
  return HKV_SUCCESS;
}

/* remove_kernel, core_kernels.cuh:679-741 */
int hkvo_erase(hkvo_table* t, uint64_t n, const uint64_t* keys) {
  {
    int drc = refuse_dual(t, "erase()", 1);
    if (drc) return drc;
  }
  for (uint64_t i = 0; i < n; i++) {
    if (is_reserved(t, keys[i])) continue;
    int64_t slot = lookup_slot(t, keys[i]);
    if (slot < 0) continue;
    t->keys[slot] = t->reclaim_key;
    t->digests[slot] = t->reclaim_digest;
    t->scores[slot] = 0;
    t->sizes[(uint64_t)slot / BUCKET]--;
  }
  return HKV_SUCCESS;
}

/* clear_kernel, core_kernels.cuh:656-676: scores and values are left as is */
int hkvo_clear(hkvo_table* t) {
  memset(t->digests, t->empty_digest, t->capacity);
  for (uint64_t i = 0; i < t->capacity; i++) t->keys[i] = t->empty_key;
  memset(t->sizes, 0, t->buckets_num * 4);
  return HKV_SUCCESS;
}

static inline int pred_eval(int pred, uint64_t key, uint64_t score,
                            uint64_t pattern, uint64_t threshold) {
  switch (pred) {
    case HKV_PRED_ALWAYS:
      return 1;
    case HKV_PRED_SCORE_LT:
      return score < threshold;
    case HKV_PRED_SCORE_LE:
      return score <= threshold;
    case HKV_PRED_SCORE_GT:
      return score > threshold;
    case HKV_PRED_SCORE_GE:
      return score >= threshold;
    case HKV_PRED_KEY_HIGH16_EQ_AND_SCORE_LT:
      return (key & UINT64_C(0xFFFF000000000000)) == pattern && score < threshold;
    default:
      return 0;
  }
}

/* dump_kernel_v2, core_kernels.cuh:983-1041; host clamp merlin_hashtable.cuh:3205-3213 */
int hkvo_export_batch_if(const hkvo_table* t, int pred, uint64_t pattern,
                         uint64_t threshold, uint64_t n, uint64_t offset,
                         uint64_t* counter, uint64_t* keys, void* values_,
                         uint64_t* scores) {
  uint8_t* values = (uint8_t*)values_;
  *counter = 0;
  if (offset >= t->capacity) return HKV_SUCCESS;
  if (n > t->capacity - offset) n = t->capacity - offset;
  uint64_t c = 0;
  for (uint64_t s = offset; s < offset + n; s++) {
    uint64_t k = t->keys[s];
    if (is_reserved(t, k)) continue;
    if (!pred_eval(pred, k, t->scores[s], pattern, threshold)) continue;
    keys[c] = k;
    if (values) memcpy(values + c * t->vb, t->values + s * t->vb, t->vb);
    if (scores) scores[c] = t->scores[s];
    c++;
  }
  *counter = c;
  return HKV_SUCCESS;
}

uint64_t hkvo_size_if(const hkvo_table* t, int pred, uint64_t pattern,
                      uint64_t threshold) {
  uint64_t c = 0;
  for (uint64_t s = 0; s < t->capacity; s++) {
    uint64_t k = t->keys[s];
    if (!is_reserved(t, k) && pred_eval(pred, k, t->scores[s], pattern, threshold)) c++;
  }
  return c;
}

/* ---- multithreaded variants (CPU baseline) --------------------------------- */

typedef struct {
  hkvo_table* t;
  uint64_t n;
  const uint64_t* keys;
  uint8_t* values;
  uint8_t* founds;
  uint64_t* scores;
  const uint64_t* in_scores;
  const uint32_t* bkts;
  uint32_t* bkts_w;
  int strategy;
  int tid, nthreads;
  int op; /* 0 = locate, 1 = find, 2 = upsert */
} mt_arg;

static void* mt_worker(void* p) {
  mt_arg* a = (mt_arg*)p;
  hkvo_table* t = a->t;
  if (a->op == 0) {
    uint64_t lo = a->n * (uint64_t)a->tid / (uint64_t)a->nthreads;
    uint64_t hi = a->n * (uint64_t)(a->tid + 1) / (uint64_t)a->nthreads;
    for (uint64_t i = lo; i < hi; i++) {
      uint64_t b;
      uint32_t s;
      uint8_t d;
      hkvo_locate(a->keys[i], t->buckets_num, &b, &s, &d);
      a->bkts_w[i] = (uint32_t)b;
    }
    return NULL;
  }
  if (a->op == 1) { /* read-only: split the batch evenly */
    uint64_t lo = a->n * (uint64_t)a->tid / (uint64_t)a->nthreads;
    uint64_t hi = a->n * (uint64_t)(a->tid + 1) / (uint64_t)a->nthreads;
    for (uint64_t i = lo; i < hi; i++)
      find_one(t, i, a->keys, a->values, a->founds, a->scores);
    return NULL;
  }
  /* writers own disjoint bucket ranges and keep input order inside them */
  uint64_t blo = t->buckets_num * (uint64_t)a->tid / (uint64_t)a->nthreads;
  uint64_t bhi = t->buckets_num * (uint64_t)(a->tid + 1) / (uint64_t)a->nthreads;
  for (uint64_t i = 0; i < a->n; i++) {
    uint32_t b = a->bkts[i];
    if (b < blo || b >= bhi) continue;
    upsert_one(t, a->strategy, i, a->keys, a->values, a->in_scores);
  }
  return NULL;
}

static void mt_run(mt_arg* proto, int threads) {
  pthread_t* th = (pthread_t*)malloc(sizeof(pthread_t) * (size_t)threads);
  mt_arg* args = (mt_arg*)malloc(sizeof(mt_arg) * (size_t)threads);
  for (int i = 0; i < threads; i++) {
    args[i] = *proto;
    args[i].tid = i;
    args[i].nthreads = threads;
    pthread_create(&th[i], NULL, mt_worker, &args[i]);
  }
  for (int i = 0; i < threads; i++) pthread_join(th[i], NULL);
  free(th);
  free(args);
}

int hkvo_find_mt(const hkvo_table* t, uint64_t n, const uint64_t* keys,
                 void* values, uint8_t* founds, uint64_t* scores, int threads) {
  if (threads <= 0) threads = hkvo_online_cores();
  mt_arg a;
  memset(&a, 0, sizeof a);
  a.t = (hkvo_table*)t;
  a.n = n;
  a.keys = keys;
  a.values = (uint8_t*)values;
  a.founds = founds;
  a.scores = scores;
  a.op = 1;
  mt_run(&a, threads);
  return HKV_SUCCESS;
}

int hkvo_insert_or_assign_mt(hkvo_table* t, uint64_t n, const uint64_t* keys,
                             const void* values, const uint64_t* scores,
                             int ignore, int threads) {
  if (n == 0) return HKV_SUCCESS;
  /* a key of a dual-bucket table has two buckets: no disjoint bucket ranges */
  if (t->dual) return hkvo_insert_or_assign(t, n, keys, values, scores, ignore);
  {
    int grc = grow_for(t, n);
    if (grc) return grc;
  }
  if (threads <= 0) threads = hkvo_online_cores();
  int strategy = strategy_of(t, ignore);
  if (!ignore) {
    int rc = check_scores_arg(t, strategy, scores);
    if (rc) return rc;
  }
  if (t->buckets_num > UINT64_C(0xFFFFFFFF))
    return fail(HKV_ERROR_UNSUPPORTED, "table too large for the mt baseline");
  uint32_t* bkts = (uint32_t*)malloc(n * 4);
  if (!bkts) return fail(HKV_ERROR_RUNTIME, "out of memory");
  mt_arg a;
  memset(&a, 0, sizeof a);
  a.t = t;
  a.n = n;
  a.keys = keys;
  a.values = (uint8_t*)values;
  a.in_scores = scores;
  a.strategy = strategy;
  a.bkts_w = bkts;
  a.op = 0;
  mt_run(&a, threads);
  a.bkts = bkts;
  a.op = 2;
  mt_run(&a, threads);
  free(bkts);
  advance_clock(t);
  return HKV_SUCCESS;
}
