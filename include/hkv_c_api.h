/*
 * C ABI of the MI355X-native bucketed key-value hash table.
 *
 * The reference (NVIDIA-Merlin/HierarchicalKV) has no FFI of its own: its
 * boundary is the C++ class template nv::merlin::HashTable<K,V,S,Strategy>
 * (include/merlin_hashtable.cuh:910-3892).  Every entry point below replaces
 * exactly one public method of that class; the citation next to each
 * declaration is the method it stands in for.  The C++ drop-in header
 * (include/merlin_hashtable.hpp) is a thin template over these symbols.
 *
 * Conventions
 *   - keys are 64-bit patterns (K = uint64_t or int64_t, reinterpreted);
 *   - scores are uint64_t;
 *   - a value row is `dim * value_size` raw bytes; only accum_or_assign does
 *     arithmetic on it (see hkv_options::value_kind);
 *   - every pointer argument must be device-accessible (HBM or pinned mapped
 *     host memory), exactly as the reference requires;
 *   - `stream` is a hipStream_t passed as void* so this header needs no HIP
 *     include; NULL is the default stream;
 *   - every function returns an hkv_status; hkv_last_error() gives the text of
 *     the last failure on the calling thread.  Status classes map one-to-one
 *     to the reference's exception types (include/merlin/debug.hpp:27-72).
 *   - calls are asynchronous with respect to the host unless stated otherwise.
 */
#ifndef HKV_C_API_H_
#define HKV_C_API_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct hkv_table hkv_table; /* opaque */
typedef void* hkv_stream_t;         /* hipStream_t */

typedef enum hkv_status {
  HKV_SUCCESS = 0,
  HKV_ERROR_CHECK = 1,    /* MERLIN_CHECK failure -> nv::merlin::MerlinException */
  HKV_ERROR_HIP = 2,      /* HIP runtime failure  -> nv::merlin::CudaException   */
  HKV_ERROR_RUNTIME = 3,  /* std::runtime_error                                   */
  HKV_ERROR_ARGUMENT = 4, /* std::invalid_argument                                */
  HKV_ERROR_UNSUPPORTED = 5 /* feature of the reference outside this build's scope */
} hkv_status;

/* nv::merlin::EvictStrategy, include/merlin_hashtable.cuh:79-87 */
typedef enum hkv_evict_strategy {
  HKV_LRU = 0,
  HKV_LFU = 1,
  HKV_EPOCH_LRU = 2,
  HKV_EPOCH_LFU = 3,
  HKV_CUSTOMIZED = 4
} hkv_evict_strategy;

/* Element type of a value row; only accum_or_assign looks at it. */
typedef enum hkv_value_kind {
  HKV_VALUE_BYTES = 0, /* opaque bytes: accum_or_assign is refused */
  HKV_VALUE_F32 = 1,
  HKV_VALUE_F64 = 2,
  HKV_VALUE_I32 = 3, /* the integer kinds add with wrap-around, signed and unsigned alike */
  HKV_VALUE_I64 = 4,
  HKV_VALUE_I8 = 5,
  HKV_VALUE_I16 = 6
} hkv_value_kind;

/* Built-in predicates for export_batch_if / size_if.  A caller that needs an
 * arbitrary device functor uses the C++ header, which instantiates the export
 * kernel on the functor against hkv_table_get_view().
 * Reference: EraseIfPredict-shaped functors, merlin_hashtable.cuh:138-179. */
typedef enum hkv_predicate {
  HKV_PRED_ALWAYS = 0,
  HKV_PRED_SCORE_LT = 1, /* score <  threshold */
  HKV_PRED_SCORE_LE = 2, /* score <= threshold */
  HKV_PRED_SCORE_GT = 3, /* score >  threshold */
  HKV_PRED_SCORE_GE = 4, /* score >= threshold */
  HKV_PRED_KEY_HIGH16_EQ_AND_SCORE_LT = 5 /* (key & 0xFFFF000000000000)==pattern && score<threshold */
} hkv_predicate;

/* nv::merlin::HashTableOptions, include/merlin_hashtable.cuh:103-136, plus the
 * three template parameters that the C ABI needs at run time. */
typedef struct hkv_options {
  uint64_t init_capacity;
  uint64_t max_capacity;
  uint64_t max_hbm_for_vectors;
  uint64_t max_bucket_size; /* only 128 is supported */
  uint64_t dim;
  float max_load_factor;
  int32_t block_size;
  int32_t io_block_size;
  int32_t device_id; /* -1: current device */
  int32_t io_by_cpu; /* host threads move the rows of insert_or_assign, find_or_insert, assign and
                        assign_values (needs max_hbm_for_vectors == 0; these calls then synchronise) */
  int32_t use_constant_memory;
  int32_t reserved_key_start_bit;
  uint64_t num_of_buckets_per_alloc;
  int32_t api_lock;
  int32_t table_mode; /* 0 = kThroughput, 1 = kMemory (dual bucket; insert_or_assign and find only) */
  /* template parameters of HashTable<K,V,S,Strategy> */
  int32_t evict_strategy; /* hkv_evict_strategy */
  int32_t value_kind;     /* hkv_value_kind */
  uint32_t value_size;    /* sizeof(V) */
  uint32_t score_size;    /* sizeof(S): 8 (the C++ header maps S = uint32_t onto it) */
} hkv_options;

/* Raw device layout of a table, for kernels compiled outside the library
 * (the C++ header's export_batch_if<Pred>).  Plain old data. */
typedef struct hkv_table_view {
  uint8_t* digests;  /* [buckets_num][128] one byte per slot                 */
  uint64_t* keys;    /* [buckets_num][128]                                   */
  uint64_t* scores;  /* [buckets_num][128]                                   */
  int32_t* sizes;    /* dual-bucket tables: [buckets_num] keys per bucket; else NULL (a
                        slot holds a key exactly when its digest is not empty_digest) */
  uint8_t* values;   /* HBM part of the value rows, slot-major               */
  uint8_t* host_values; /* pinned host part (hybrid mode) or NULL            */
  uint64_t hbm_slots;   /* slots [0,hbm_slots) live in `values`, the rest in
                           `host_values` starting at slot hbm_slots           */
  uint64_t buckets_num;
  uint64_t capacity;    /* buckets_num * 128 */
  uint32_t value_bytes; /* dim * value_size */
  uint32_t dim;
  uint64_t empty_key, reclaim_key, locked_key;
  uint64_t reserved_mask1, reserved_mask2; /* reserved <=> (k & mask1) == mask2 */
  uint8_t empty_digest, reclaim_digest;
  uint8_t pow2_buckets; /* buckets_num is a power of two */
  uint8_t dual_bucket;  /* TableMode::kMemory: a key lives in one of two buckets */
  uint8_t pad_[4];
  uint64_t* bounds;     /* NULL for dual-bucket tables.  [buckets_num][8]: for each run of 16
                           slots a value that is not above any score in it (0 is always right); kept
                           tight by the upserts, which with it read one or two of a bucket's
                           eight score lines instead of all of them.  Whoever lowers a score
                           in place sets the bound of its run to 0 or calls
                           hkv_scores_changed */
} hkv_table_view;

/* BaseAllocator (include/merlin/allocator.cuh:27-58) as a table of callbacks.
 * memory_type: 0 = Device, 1 = Pinned (host, device-mapped), 2 = Host.
 * Both callbacks return 0 on success.  A table created with an allocator
 * takes every byte of table memory from it. */
typedef struct hkv_allocator {
  void* ctx;
  int (*alloc)(void* ctx, int memory_type, void** ptr, size_t size);
  int (*free)(void* ctx, int memory_type, void* ptr);
} hkv_allocator;

/* Fill `opts` with the defaults of HashTableOptions (merlin_hashtable.cuh:103-136),
 * K=uint64, V=float, S=uint64, LRU. */
void hkv_options_default(hkv_options* opts);

/* Text of the last error on this thread (the reference throws: debug.hpp:27-72). */
const char* hkv_last_error(void);
/* Version string of the library, and the gfx target it was compiled for (no counterpart in
 * the reference). */
const char* hkv_version(void);

/* HashTable::init, merlin_hashtable.cuh:984-1085 (+ create_table,
 * core_kernels.cuh:327-381).  Synchronous. */
int hkv_table_create(const hkv_options* opts, hkv_table** out);
/* HashTable::init with a caller-supplied allocator (same lines). */
int hkv_table_create_with_allocator(const hkv_options* opts,
                                    const hkv_allocator* allocator,
                                    hkv_table** out);
/* HashTable::~HashTable, merlin_hashtable.cuh:953-971.  Synchronous. */
int hkv_table_destroy(hkv_table* t);

/* unique_key (here and below): 1 = the caller guarantees that no key occurs twice in the
 * batch; 0 = keys may repeat: the batch is first reduced to one occurrence per key (device
 * sort, temporary memory from the stream's pool), as the reference's kernels for such
 * batches leave every key in the table once.  A dual-bucket table needs 1
 * (merlin_hashtable.cuh:1167-1169).
 *
 * HashTable::insert_or_assign, merlin_hashtable.cuh:1125-1305.  On a table with rows in host
 * memory and with unique_key = 1 (the reference's lock-key and write kernels, upsert.cuh:1350-1595)
 * every slot a key of the batch takes stays locked until all keys of the batch are settled: no
 * key takes the slot of another key of its batch, and a key whose score is not above the lowest
 * score still visible in its bucket is refused.  find_or_insert with values does the same. */
int hkv_insert_or_assign(hkv_table* t, uint64_t n, const uint64_t* keys,
                         const void* values, const uint64_t* scores,
                         hkv_stream_t stream, int unique_key,
                         int ignore_evict_strategy);

/* insert_or_assign for callers that cannot allocate device memory (code under HIP graph
 * capture, serving loops and harnesses that forbid hipMalloc).  No counterpart in the
 * reference.  Same results as hkv_insert_or_assign with unique_key = 1, through the two-phase
 * path: its scratch (one 32-bit list head per bucket, one link per key) lives in a device array
 * that is part of the library image, 8 MiB per GPU, held until the process ends, instead of
 * memory allocated by the call; the call itself allocates nothing.
 * Limits: n <= 2^20 keys per call, tables of up to 2^20 buckets (capacity 2^27), keys unique in
 * the batch, a table that cannot grow any more (init_capacity * 2 > max_capacity, or grown to the
 * maximum), api_lock on, no io_by_cpu, no dual-bucket mode, no keys held by lock_keys: anything
 * else is refused with HKV_ERROR_ARGUMENT / HKV_ERROR_UNSUPPORTED and a message.
 * All calls on one GPU share that GPU's array (also across tables): calls that overlap in time on
 * one GPU race on it; calls on one stream, or ordered by the group lock of one table, do not. */
int hkv_insert_or_assign_noalloc(hkv_table* t, uint64_t n, const uint64_t* keys,
                                 const void* values, const uint64_t* scores,
                                 hkv_stream_t stream, int ignore_evict_strategy);

/* HashTable::insert_and_evict (device counter overload),
 * merlin_hashtable.cuh:1351-1473.  The caller zeroes *d_evicted_counter. */
int hkv_insert_and_evict(hkv_table* t, uint64_t n, const uint64_t* keys,
                         const void* values, const uint64_t* scores,
                         uint64_t* evicted_keys, void* evicted_values,
                         uint64_t* evicted_scores, uint64_t* d_evicted_counter,
                         hkv_stream_t stream, int unique_key,
                         int ignore_evict_strategy);

/* HashTable::insert_and_evict (count-returning overload),
 * merlin_hashtable.cuh:1518-1546.  Synchronises `stream`. */
int hkv_insert_and_evict_count(hkv_table* t, uint64_t n, const uint64_t* keys,
                               const void* values, const uint64_t* scores,
                               uint64_t* evicted_keys, void* evicted_values,
                               uint64_t* evicted_scores, hkv_stream_t stream,
                               int unique_key, int ignore_evict_strategy,
                               uint64_t* n_evicted);

/* HashTable::accum_or_assign, merlin_hashtable.cuh:1589-1680 */
int hkv_accum_or_assign(hkv_table* t, uint64_t n, const uint64_t* keys,
                        const void* value_or_deltas,
                        const uint8_t* accum_or_assigns /* bool[n] */,
                        const uint64_t* scores, hkv_stream_t stream,
                        int ignore_evict_strategy);

/* HashTable::find_or_insert (value overload), merlin_hashtable.cuh:1699-1857.
 * `values` is in-out; `scores` is input only (as in the reference kernels). */
int hkv_find_or_insert(hkv_table* t, uint64_t n, const uint64_t* keys,
                       void* values, const uint64_t* scores,
                       hkv_stream_t stream, int unique_key,
                       int ignore_evict_strategy);

/* HashTable::find_or_insert (pointer overload), merlin_hashtable.cuh:1883-1966 */
int hkv_find_or_insert_ptr(hkv_table* t, uint64_t n, const uint64_t* keys,
                           void** values, uint8_t* founds /* bool[n] */,
                           const uint64_t* scores, hkv_stream_t stream,
                           int unique_key, int ignore_evict_strategy);
/* The same overload with locked_key_ptrs (merlin_hashtable.cuh:1878-1927,
 * find_ptr_or_insert.cuh:27-245): the slots of the accepted keys stay LOCKED, their key
 * addresses are returned, and the caller releases them with hkv_unlock_keys after writing
 * the rows.  Keys of the batch must be unique. */
int hkv_find_or_insert_ptr_lock(hkv_table* t, uint64_t n, const uint64_t* keys,
                                void** values, uint8_t* founds, const uint64_t* scores,
                                uint64_t** locked_key_ptrs, hkv_stream_t stream,
                                int ignore_evict_strategy);

/* HashTable::assign (values + scores), merlin_hashtable.cuh:2071-2213 */
int hkv_assign(hkv_table* t, uint64_t n, const uint64_t* keys,
               const void* values, const uint64_t* scores, hkv_stream_t stream,
               int unique_key);
/* HashTable::assign_scores, merlin_hashtable.cuh:2228-2283 */
int hkv_assign_scores(hkv_table* t, uint64_t n, const uint64_t* keys,
                      const uint64_t* scores, hkv_stream_t stream,
                      int unique_key);
/* HashTable::assign_values, merlin_hashtable.cuh:2299-2444 */
int hkv_assign_values(hkv_table* t, uint64_t n, const uint64_t* keys,
                      const void* values, hkv_stream_t stream, int unique_key);

/* HashTable::find (founds overload), merlin_hashtable.cuh:2464-2577 */
int hkv_find(const hkv_table* t, uint64_t n, const uint64_t* keys, void* values,
             uint8_t* founds /* bool[n] */, uint64_t* scores,
             hkv_stream_t stream);
/* HashTable::find (missed-keys overload), merlin_hashtable.cuh:2600-2705 */
int hkv_find_missed(const hkv_table* t, uint64_t n, const uint64_t* keys,
                    void* values, uint64_t* missed_keys, int32_t* missed_indices,
                    int32_t* missed_size, uint64_t* scores, hkv_stream_t stream);
/* HashTable::find (pointer overload, "find*"), merlin_hashtable.cuh:2729-2795 */
int hkv_find_ptr(const hkv_table* t, uint64_t n, const uint64_t* keys,
                 void** values, uint8_t* founds /* bool[n] */, uint64_t* scores,
                 hkv_stream_t stream, int unique_key);
/* HashTable::contains, merlin_hashtable.cuh:2856-2894 */
int hkv_contains(const hkv_table* t, uint64_t n, const uint64_t* keys,
                 uint8_t* founds /* bool[n] */, hkv_stream_t stream);

/* HashTable::lock_keys, merlin_hashtable.cuh:1982-2012: every key that is
 * present has its key word set to LOCKED and its score touched;
 * locked_key_ptrs[i] = address of that key word, or null.  While keys are
 * locked they are invisible to lookups, and slots holding them are never
 * chosen as eviction victims.  Unlike the reference, the `scores` argument is
 * checked against the eviction strategy as in the other calls. */
int hkv_lock_keys(hkv_table* t, uint64_t n, const uint64_t* keys,
                  uint64_t** locked_key_ptrs, uint8_t* success /* bool[n], may be null */,
                  const uint64_t* scores, hkv_stream_t stream);
/* HashTable::unlock_keys, merlin_hashtable.cuh:2026-2044 */
int hkv_unlock_keys(hkv_table* t, uint64_t n, uint64_t** locked_key_ptrs,
                    const uint64_t* keys, uint8_t* success /* may be null */,
                    hkv_stream_t stream);
/* HashTable::find_and_update, merlin_hashtable.cuh:2811-2843: find* that also
 * touches the score of every key it finds; with `scores` given, scores[i] is
 * the input of the score rule and receives the score after the touch. */
int hkv_find_and_update(hkv_table* t, uint64_t n, const uint64_t* keys,
                        void** values, uint8_t* founds, uint64_t* scores,
                        hkv_stream_t stream);

/* HashTable::erase, merlin_hashtable.cuh:2904-2930 */
int hkv_erase(hkv_table* t, uint64_t n, const uint64_t* keys,
              hkv_stream_t stream);
/* HashTable::clear, merlin_hashtable.cuh:3059-3078 */
int hkv_clear(hkv_table* t, hkv_stream_t stream);
/* HashTable::reserve, merlin_hashtable.cuh:3503-3541: doubles the bucket count
 * (rehash) until capacity >= new_capacity or max_capacity would be passed.
 * Tables created with init_capacity * 2 <= max_capacity also grow by
 * themselves at the head of every inserting call, as the reference's do
 * (merlin_hashtable.cuh:1151-1154).  Synchronises the device. */
int hkv_reserve(hkv_table* t, uint64_t new_capacity, hkv_stream_t stream);
/* HashTable::set_max_capacity, merlin_hashtable.cuh:3561-3579: a power of two;
 * values below the current capacity are ignored; growth is possible again. */
int hkv_set_max_capacity(hkv_table* t, uint64_t new_max_capacity);

/* HashTable::export_batch (device counter), merlin_hashtable.cuh:3099-3147 */
int hkv_export_batch(const hkv_table* t, uint64_t n, uint64_t offset,
                     uint64_t* d_counter, uint64_t* keys, void* values,
                     uint64_t* scores, hkv_stream_t stream);
/* HashTable::export_batch_if<Pred>, merlin_hashtable.cuh:3193-3276, with one of
 * the built-in predicates. */
int hkv_export_batch_if(const hkv_table* t, int predicate, uint64_t pattern,
                        uint64_t threshold, uint64_t n, uint64_t offset,
                        uint64_t* d_counter, uint64_t* keys, void* values,
                        uint64_t* scores, hkv_stream_t stream);
/* HashTable::size_if<Pred>, merlin_hashtable.cuh:3460-3476.  Synchronises. */
int hkv_size_if(const hkv_table* t, int predicate, uint64_t pattern,
                uint64_t threshold, hkv_stream_t stream, uint64_t* out);

/* HashTable::size, merlin_hashtable.cuh:3424-3451.  Synchronises `stream`. */
int hkv_size(const hkv_table* t, hkv_stream_t stream, uint64_t* out);
/* HashTable::empty merlin_hashtable.cuh:3416, capacity :3487, load_factor :3551, dim :3586,
 * max_bucket_size :3593, bucket_count :3602 (same file) */
int hkv_empty(const hkv_table* t, hkv_stream_t stream, int* out);
uint64_t hkv_capacity(const hkv_table* t);
int hkv_load_factor(const hkv_table* t, hkv_stream_t stream, float* out);
uint64_t hkv_dim(const hkv_table* t);
uint64_t hkv_max_bucket_size(const hkv_table* t);
uint64_t hkv_bucket_count(const hkv_table* t);
/* 1 when every value row lives in HBM (Table::is_pure_hbm, types.cuh:195-220) */
int hkv_is_pure_hbm(const hkv_table* t);

/* HashTable::set_global_epoch, merlin_hashtable.cuh:3760-3762 */
int hkv_set_global_epoch(hkv_table* t, uint64_t epoch);

/* Layout handle for kernels compiled by the caller (C++ header): what the reference's
 * templates read from Table<K,V,S> directly (types.cuh:178-220). */
int hkv_table_get_view(const hkv_table* t, hkv_table_view* out);
/* The C++ header brackets a caller-compiled kernel with the table's group
 * lock (group_lock.cuh:217-337): role 0 = reader, 1 = updater, 2 = inserter.
 * begin orders `stream` after every conflicting operation already enqueued;
 * end publishes the work enqueued on `stream` since begin. */
int hkv_lock_begin(const hkv_table* t, int role, hkv_stream_t stream);
int hkv_lock_end(const hkv_table* t, int role, hkv_stream_t stream);

/* Clock used by the LRU / EpochLRU strategies (device_nano, utils.cuh:75-80).
 *   mode 0: hardware clock, nanoseconds (default);
 *   mode 1: deterministic: the key at batch index i sees
 *           now = base + (i << 20); after every mutating call base advances
 *           by 2^40.  Makes LRU scores reproducible for parity tests; the
 *           reference's own tests can only bound them (no counterpart there).
 */
int hkv_set_clock(hkv_table* t, int mode, uint64_t base);

/* Scores may have been changed by code outside the library: a functor handed to for_each gets
 * a writable score (merlin_hashtable.cuh:3372-3412).  The table then drops what it knows about
 * the scores (hkv_table_view::bounds) before it relies on it again.  No counterpart in the
 * reference, which keeps no such knowledge. */
int hkv_scores_changed(hkv_table* t);

/* Measurement aid, no counterpart in the reference (its benchmark times whole calls on the host,
 * benchmark/merlin_hashtable_benchmark.cc.cu:166-265): the next find or upsert-family call made
 * by the calling thread launches its kernel with these two HIP events (hipEvent_t, created by the
 * caller), which the runtime stamps with the start and the end of that kernel's execution;
 * hipEventElapsedTime(start, stop) is then the kernel's own duration, as a profiler reports it.
 * Two null pointers cancel a pending request. */
int hkv_time_next_kernel(void* start_event, void* stop_event);

#ifdef __cplusplus
}
#endif
#endif /* HKV_C_API_H_ */
