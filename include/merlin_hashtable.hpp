/*
 * Source-level drop-in for the reference's public header
 * (include/merlin_hashtable.cuh): the same namespace, class names, method
 * names, parameter order and defaults, with hipStream_t where the reference
 * has cudaStream_t.  Every method forwards to one entry point of the C ABI
 * (include/hkv_c_api.h) of libhkv.so; only the predicate templates
 * (export_batch_if, size_if, erase_if) instantiate a kernel in the caller's
 * translation unit, against the table layout of hkv_table_get_view().
 *
 * Compile with hipcc for gfx950 and link with -lhkv.
 *
 * Reference lines mirrored here:
 *   EvictStrategy ........ merlin_hashtable.cuh:79-87
 *   TableMode ............ merlin_hashtable.cuh:95-98
 *   HashTableOptions ..... merlin_hashtable.cuh:103-136
 *   HashTableBase ........ merlin_hashtable.cuh:187-885
 *   HashTable ............ merlin_hashtable.cuh:910-3892
 *   MemoryType, BaseAllocator, DefaultAllocator .. merlin/allocator.cuh:27-125
 *   BaseKVFile ........... merlin/types.cuh:242-281
 *   exceptions, checks ... merlin/debug.hpp:27-72
 *   GB / MB / KB ......... merlin/utils.cuh:338-342
 *
 * TableMode::kMemory (dual bucket) runs insert_or_assign, find, clear, size and
 * the export family, as in the reference; the calls the reference guards throw
 * the same way, and assign, find*, lock_keys / unlock_keys / find_and_update
 * (unguarded but single-bucket in the reference) throw too.
 * Buckets have 128 slots: init() throws for any other max_bucket_size (the reference takes
 * powers of two from 8 to 2048; 128 is its default and the length its tuned kernels assume).
 * S = uint32_t (Customized strategy only, as in the reference) is served by widening and
 * narrowing the caller's score arrays around each call: the table keeps 64-bit scores, and
 * such calls allocate a temporary buffer on the stream.
 */
#ifndef MERLIN_HASHTABLE_HPP_
#define MERLIN_HASHTABLE_HPP_

#include <hip/hip_cooperative_groups.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <limits>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

#include "hkv_c_api.h"
#include "hkv_device.hpp"

/* as merlin/utils.cuh:30: caller functors name the tile type cg::thread_block_tile<N>;
 * the namespace behind the alias is cooperative_groups plus pointer shuffles */
namespace cg = hkv::coop;

namespace nv {
namespace merlin {

/* ---- merlin/debug.hpp ------------------------------------------------------- */

class CudaException : public std::runtime_error {
 public:
  CudaException(const std::string& what) : runtime_error(what) {}
};

class MerlinException : public std::runtime_error {
 public:
  MerlinException(const std::string& what) : runtime_error(what) {}
};

inline void hip_check_(hipError_t val, const char* file, int line) {
  if (val != hipSuccess) {
    std::ostringstream os;
    os << file << ':' << line << ": HIP error " << hipGetErrorName(val) << " (#" << val
       << "): " << hipGetErrorString(val);
    throw CudaException(os.str());
  }
}
#define HKV_HIP_CHECK(val) ::nv::merlin::hip_check_((val), __FILE__, __LINE__)

template <class Msg>
inline void merlin_check_(bool cond, const Msg& msg, const char* file, int line) {
  if (!cond) {
    std::ostringstream os;
    os << file << ':' << line << ": HierarchicalKV error " << msg;
    throw MerlinException(os.str());
  }
}
#ifndef MERLIN_CHECK
#define MERLIN_CHECK(cond, msg) ::nv::merlin::merlin_check_((cond), (msg), __FILE__, __LINE__)
#endif

/* status of a C ABI call -> the exception the reference would have thrown */
inline void throw_on_error_(int rc) {
  if (rc == HKV_SUCCESS) return;
  const std::string msg = hkv_last_error();
  switch (rc) {
    case HKV_ERROR_CHECK:
      throw MerlinException(msg);
    case HKV_ERROR_HIP:
      throw CudaException(msg);
    case HKV_ERROR_ARGUMENT:
      throw std::invalid_argument(msg);
    default:
      throw std::runtime_error(msg);
  }
}

/* ---- merlin/utils.cuh --------------------------------------------------------- */

static inline size_t GB(size_t n) { return n << 30; }
static inline size_t MB(size_t n) { return n << 20; }
static inline size_t KB(size_t n) { return n << 10; }

/* ---- merlin/allocator.cuh ------------------------------------------------------ */

enum MemoryType {
  Device,   // HBM
  Pinned,   // Pinned Host Memory
  Host,     // Host Memory
  Managed,  // Pageable Host Memory(Not required)
};

class BaseAllocator {
 public:
  BaseAllocator(const BaseAllocator&) = delete;
  BaseAllocator(BaseAllocator&&) = delete;
  BaseAllocator& operator=(const BaseAllocator&) = delete;
  BaseAllocator& operator=(BaseAllocator&&) = delete;
  BaseAllocator() = default;
  virtual ~BaseAllocator() = default;

  virtual void alloc(const MemoryType type, void** ptr, size_t size,
                     unsigned int pinned_flags = hipHostMallocDefault) = 0;
  virtual void alloc_async(const MemoryType type, void** ptr, size_t size,
                           hipStream_t stream) = 0;
  virtual void free(const MemoryType type, void* ptr) = 0;
  virtual void free_async(const MemoryType type, void* ptr, hipStream_t stream) = 0;
};

class DefaultAllocator : public virtual BaseAllocator {
 public:
  DefaultAllocator() {}
  ~DefaultAllocator() override {}

  void alloc(const MemoryType type, void** ptr, size_t size,
             unsigned int pinned_flags = hipHostMallocDefault) override {
    switch (type) {
      case MemoryType::Device:
        HKV_HIP_CHECK(hipMalloc(ptr, size));
        break;
      case MemoryType::Pinned:
        HKV_HIP_CHECK(hipHostMalloc(ptr, size, pinned_flags));
        break;
      case MemoryType::Host:
        *ptr = std::malloc(size);
        break;
      default:
        throw std::runtime_error("Unsupported memory type.");
    }
  }
  void alloc_async(const MemoryType type, void** ptr, size_t size, hipStream_t stream) override {
    if (type == MemoryType::Device) {
      HKV_HIP_CHECK(hipMallocAsync(ptr, size, stream));
    } else {
      throw std::runtime_error("Only support async allocation on HBM.");
    }
  }
  void free(const MemoryType type, void* ptr) override {
    if (ptr == nullptr) return;
    switch (type) {
      case MemoryType::Pinned:
        HKV_HIP_CHECK(hipHostFree(ptr));
        break;
      case MemoryType::Device:
        HKV_HIP_CHECK(hipFree(ptr));
        break;
      case MemoryType::Host:
        std::free(ptr);
        break;
      default:
        throw std::runtime_error("Unsupported memory type.");
    }
  }
  void free_async(const MemoryType type, void* ptr, hipStream_t stream) override {
    if (ptr == nullptr) return;
    if (type == MemoryType::Device) {
      HKV_HIP_CHECK(hipFreeAsync(ptr, stream));
    } else {
      throw std::runtime_error("Only support async free on HBM.");
    }
  }
};

/* ---- merlin/types.cuh ------------------------------------------------------------ */

template <class K, class V, class S>
class BaseKVFile {
 public:
  virtual ~BaseKVFile() {}
  virtual size_t read(const size_t n, const size_t dim, K* keys, V* vectors, S* scores) = 0;
  virtual size_t write(const size_t n, const size_t dim, const K* keys, const V* vectors,
                       const S* scores) = 0;
};

/* ---- merlin_hashtable.cuh ---------------------------------------------------------- */

struct EvictStrategy {
  enum EvictStrategyEnum {
    kLru = 0,         ///< LRU mode.
    kLfu = 1,         ///< LFU mode.
    kEpochLru = 2,    ///< Epoch Lru mode.
    kEpochLfu = 3,    ///< Epoch Lfu mode.
    kCustomized = 4,  ///< Customized mode.
  };
};

enum class TableMode {
  kThroughput = 0,  ///< Default: single-bucket, max throughput.
  kMemory = 1,      ///< Dual-bucket, higher load factor.
};

/* memory_pool.cuh:139-143; kept so option structs copy over unchanged.  The
 * library takes its few scratch words from the table allocation instead. */
struct MemoryPoolOptions {
  size_t max_stock = 4;
  size_t max_pending = 16;
};

struct HashTableOptions {
  size_t init_capacity = 0;        ///< The initial capacity of the hash table.
  size_t max_capacity = 0;         ///< The maximum capacity of the hash table.
  size_t max_hbm_for_vectors = 0;  ///< The maximum HBM for vectors, in bytes.
  size_t max_bucket_size = 128;    ///< The length of each bucket (only 128 here).
  size_t dim = 64;                 ///< The dimension of the vectors.
  float max_load_factor = 0.5f;    ///< The max load factor before rehashing.
  int block_size = 128;            ///< Kept for source compatibility; unused.
  int io_block_size = 1024;        ///< Kept for source compatibility; unused.
  int device_id = -1;              ///< The ID of device.
  bool io_by_cpu = false;          ///< Host threads move the rows of the writers (needs max_hbm_for_vectors == 0).
  bool use_constant_memory = false;  ///< reserved
  int reserved_key_start_bit = 0;       ///< The binary index of reserved key.
  size_t num_of_buckets_per_alloc = 1;  ///< Checked as in the reference; the
                                        ///< table is one arena whatever it says.
  bool api_lock = true;  ///< Order calls on different streams by role.
  TableMode table_mode = TableMode::kThroughput;
  MemoryPoolOptions device_memory_pool;
  MemoryPoolOptions host_memory_pool;
};

template <class K, class S>
using EraseIfPredict = bool (*)(const K& key, S& score, const K& pattern, const S& threshold);

template <typename K, typename V, typename S = uint64_t>
class HashTableBase {
 public:
  using size_type = size_t;
  using key_type = K;
  using value_type = V;
  using score_type = S;
  using allocator_type = BaseAllocator;

  virtual ~HashTableBase() {}
  virtual void init(const HashTableOptions& options, allocator_type* allocator = nullptr) = 0;
  virtual void insert_or_assign(const size_type n, const key_type* keys, const value_type* values,
                                const score_type* scores = nullptr, hipStream_t stream = 0,
                                bool unique_key = true, bool ignore_evict_strategy = false) = 0;
  virtual void insert_and_evict(const size_type n, const key_type* keys, const value_type* values,
                                const score_type* scores, key_type* evicted_keys,
                                value_type* evicted_values, score_type* evicted_scores,
                                size_type* d_evicted_counter, hipStream_t stream = 0,
                                bool unique_key = true, bool ignore_evict_strategy = false) = 0;
  virtual size_type insert_and_evict(const size_type n, const key_type* keys,
                                     const value_type* values, const score_type* scores,
                                     key_type* evicted_keys, value_type* evicted_values,
                                     score_type* evicted_scores, hipStream_t stream = 0,
                                     bool unique_key = true,
                                     bool ignore_evict_strategy = false) = 0;
  virtual void accum_or_assign(const size_type n, const key_type* keys,
                               const value_type* value_or_deltas, const bool* accum_or_assigns,
                               const score_type* scores = nullptr, hipStream_t stream = 0,
                               bool ignore_evict_strategy = false) = 0;
  virtual void find_or_insert(const size_type n, const key_type* keys, value_type* values,
                              score_type* scores = nullptr, hipStream_t stream = 0,
                              bool unique_key = true, bool ignore_evict_strategy = false) = 0;
  virtual void find_or_insert(const size_type n, const key_type* keys, value_type** values,
                              bool* founds, score_type* scores = nullptr, hipStream_t stream = 0,
                              bool unique_key = true, bool ignore_evict_strategy = false,
                              key_type** locked_key_ptrs = nullptr) = 0;
  virtual void lock_keys(const size_type n, key_type const* keys, key_type** locked_key_ptrs,
                         bool* succeededs = nullptr, hipStream_t stream = 0,
                         score_type const* scores = nullptr) = 0;
  virtual void unlock_keys(const size_type n, key_type** locked_key_ptrs, const key_type* keys,
                           bool* succeededs = nullptr, hipStream_t stream = 0) = 0;
  virtual void assign(const size_type n, const key_type* keys, const value_type* values,
                      const score_type* scores = nullptr, hipStream_t stream = 0,
                      bool unique_key = true) = 0;
  virtual void assign_scores(const size_type n, const key_type* keys,
                             const score_type* scores = nullptr, hipStream_t stream = 0,
                             bool unique_key = true) = 0;
  virtual void assign(const size_type n, const key_type* keys, const score_type* scores = nullptr,
                      hipStream_t stream = 0, bool unique_key = true) = 0;
  virtual void assign_values(const size_type n, const key_type* keys, const value_type* values,
                             hipStream_t stream = 0, bool unique_key = true) = 0;
  virtual void find(const size_type n, const key_type* keys, value_type* values, bool* founds,
                    score_type* scores = nullptr, hipStream_t stream = 0) const = 0;
  virtual void find(const size_type n, const key_type* keys, value_type* values,
                    key_type* missed_keys, int* missed_indices, int* missed_size,
                    score_type* scores = nullptr, hipStream_t stream = 0) const = 0;
  virtual void find(const size_type n, const key_type* keys, value_type** values, bool* founds,
                    score_type* scores = nullptr, hipStream_t stream = 0,
                    bool unique_key = true) const = 0;
  virtual void find_and_update(const size_type n, const key_type* keys, value_type** values,
                               bool* founds, score_type* scores = nullptr, hipStream_t stream = 0,
                               bool unique_key = true) = 0;
  virtual void contains(const size_type n, const key_type* keys, bool* founds,
                        hipStream_t stream = 0) const = 0;
  virtual void erase(const size_type n, const key_type* keys, hipStream_t stream = 0) = 0;
  virtual void clear(hipStream_t stream = 0) = 0;
  virtual void export_batch(size_type n, const size_type offset, size_type* d_counter,
                            key_type* keys, value_type* values, score_type* scores = nullptr,
                            hipStream_t stream = 0) const = 0;
  virtual size_type export_batch(const size_type n, const size_type offset, key_type* keys,
                                 value_type* values, score_type* scores = nullptr,
                                 hipStream_t stream = 0) const = 0;
  virtual bool empty(hipStream_t stream = 0) const = 0;
  virtual size_type size(hipStream_t stream = 0) const = 0;
  virtual size_type capacity() const = 0;
  virtual void reserve(const size_type new_capacity, hipStream_t stream = 0) = 0;
  virtual float load_factor(hipStream_t stream = 0) const = 0;
  virtual void set_max_capacity(size_type new_max_capacity) = 0;
  virtual size_type dim() const noexcept = 0;
  virtual size_type max_bucket_size() const noexcept = 0;
  virtual size_type bucket_count() const noexcept = 0;
  virtual size_type save(BaseKVFile<K, V, S>* file,
                         const size_t max_workspace_size = 1L * 1024 * 1024,
                         hipStream_t stream = 0) const = 0;
  virtual size_type load(BaseKVFile<K, V, S>* file,
                         const size_t max_workspace_size = 1L * 1024 * 1024,
                         hipStream_t stream = 0) = 0;
  virtual void set_global_epoch(const uint64_t epoch) = 0;
};

namespace detail {

template <class V>
constexpr int value_kind_of() {
  if (std::is_same<V, float>::value) return HKV_VALUE_F32;
  if (std::is_same<V, double>::value) return HKV_VALUE_F64;
  if (std::is_same<V, int32_t>::value || std::is_same<V, uint32_t>::value) return HKV_VALUE_I32;
  if (std::is_same<V, int64_t>::value || std::is_same<V, uint64_t>::value) return HKV_VALUE_I64;
  if (std::is_same<V, int8_t>::value || std::is_same<V, uint8_t>::value) return HKV_VALUE_I8;
  if (std::is_same<V, int16_t>::value || std::is_same<V, uint16_t>::value) return HKV_VALUE_I16;
  return HKV_VALUE_BYTES;
}

/* Score arrays at the boundary.  The C ABI speaks 64-bit scores; for S = uint64_t these
 * wrappers are the caller's pointer, for S = uint32_t a temporary 64-bit array on the
 * stream that is filled from / written back to the caller's 32-bit array. */
template <class S>
struct ScoresIn {
  const uint64_t* p;
  ScoresIn(const S* s, size_t, hipStream_t) : p(s) {}
  const uint64_t* get() const { return p; }
};
template <>
struct ScoresIn<uint32_t> {
  uint64_t* tmp = nullptr;
  hipStream_t st;
  ScoresIn(const uint32_t* s, size_t n, hipStream_t stream) : st(stream) {
    if (s == nullptr || n == 0) return;
    HKV_HIP_CHECK(hipMallocAsync(reinterpret_cast<void**>(&tmp), n * sizeof(uint64_t), st));
    hipLaunchKernelGGL(hkv::widen_scores_kernel, dim3(static_cast<unsigned>((n + 255) / 256)),
                       dim3(256), 0, st, s, tmp, static_cast<uint64_t>(n));
  }
  ~ScoresIn() {
    if (tmp) (void)hipFreeAsync(tmp, st);
  }
  ScoresIn(const ScoresIn&) = delete;
  ScoresIn& operator=(const ScoresIn&) = delete;
  const uint64_t* get() const { return tmp; }
};
template <class S>
struct ScoresOut {
  uint64_t* p;
  ScoresOut(S* s, size_t, hipStream_t) : p(s) {}
  uint64_t* get() const { return p; }
  void finish() {}
};
template <>
struct ScoresOut<uint32_t> {
  uint32_t* dst;
  uint64_t* tmp = nullptr;
  size_t n;
  hipStream_t st;
  /* starts from the caller's contents: entries a call leaves untouched (keys not found)
   * come back unchanged */
  ScoresOut(uint32_t* s, size_t n_, hipStream_t stream) : dst(s), n(n_), st(stream) {
    if (s == nullptr || n == 0) return;
    HKV_HIP_CHECK(hipMallocAsync(reinterpret_cast<void**>(&tmp), n * sizeof(uint64_t), st));
    hipLaunchKernelGGL(hkv::widen_scores_kernel, dim3(static_cast<unsigned>((n + 255) / 256)),
                       dim3(256), 0, st, s, tmp, static_cast<uint64_t>(n));
  }
  ~ScoresOut() {
    if (tmp) (void)hipFreeAsync(tmp, st);
  }
  ScoresOut(const ScoresOut&) = delete;
  ScoresOut& operator=(const ScoresOut&) = delete;
  uint64_t* get() const { return tmp; }
  void finish() {
    if (tmp)
      hipLaunchKernelGGL(hkv::narrow_scores_kernel, dim3(static_cast<unsigned>((n + 255) / 256)),
                         dim3(256), 0, st, tmp, dst, static_cast<uint64_t>(n));
  }
};

/* the caller's functor sees K and S; the kernel works on the 64-bit patterns */
template <class K, class S, template <typename, typename> class PredFunctor>
struct PredAdapter {
  __device__ __forceinline__ bool operator()(const uint64_t& key, uint64_t& score,
                                             const uint64_t& pattern,
                                             const uint64_t& threshold) const {
    PredFunctor<K, S> pred;
    const K k = static_cast<K>(key);
    S s = static_cast<S>(score);
    const K p = static_cast<K>(pattern);
    const S t = static_cast<S>(threshold);
    return pred(k, s, p, t);
  }
};

inline int alloc_cb(void* ctx, int type, void** ptr, size_t size) {
  try {
    static_cast<BaseAllocator*>(ctx)->alloc(static_cast<MemoryType>(type), ptr, size,
                                            hipHostMallocMapped | hipHostMallocPortable);
    return 0;
  } catch (...) {
    return 1;
  }
}
inline int free_cb(void* ctx, int type, void* ptr) {
  try {
    static_cast<BaseAllocator*>(ctx)->free(static_cast<MemoryType>(type), ptr);
    return 0;
  } catch (...) {
    return 1;
  }
}

/* A staging array of save / load: device memory or pinned host memory, freed by the destructor. */
template <class T>
class StageBuffer {
 public:
  StageBuffer(size_t count, bool pinned_host) : host_(pinned_host) {
    void* p = nullptr;
    if (host_)
      HKV_HIP_CHECK(hipHostMalloc(&p, count * sizeof(T)));
    else
      HKV_HIP_CHECK(hipMalloc(&p, count * sizeof(T)));
    p_ = static_cast<T*>(p);
  }
  ~StageBuffer() {
    if (p_ == nullptr) return;
    if (host_)
      (void)hipHostFree(p_);
    else
      (void)hipFree(p_);
  }
  StageBuffer(const StageBuffer&) = delete;
  StageBuffer& operator=(const StageBuffer&) = delete;
  T* get() const { return p_; }

 private:
  bool host_;
  T* p_ = nullptr;
};

/* One device word from the stream-ordered allocator for a call that returns a count; given
 * back on every way out of the call. */
template <class T>
class DeviceWord {
 public:
  explicit DeviceWord(hipStream_t s) : s_(s) {
    HKV_HIP_CHECK(hipMallocAsync(reinterpret_cast<void**>(&p_), sizeof(T), s_));
  }
  ~DeviceWord() {
    if (p_ != nullptr) (void)hipFreeAsync(p_, s_);
  }
  DeviceWord(const DeviceWord&) = delete;
  DeviceWord& operator=(const DeviceWord&) = delete;
  T* get() const { return p_; }
  /* the word's value once the stream has run everything enqueued so far */
  T read() const {
    T h{};
    HKV_HIP_CHECK(hipMemcpyAsync(&h, p_, sizeof h, hipMemcpyDeviceToHost, s_));
    HKV_HIP_CHECK(hipStreamSynchronize(s_));
    return h;
  }

 private:
  hipStream_t s_;
  T* p_ = nullptr;
};

/* RAII bracket of the table's group lock around a caller-compiled kernel */
struct RoleGuard {
  const hkv_table* t;
  int role;
  hipStream_t s;
  RoleGuard(const hkv_table* t_, int role_, hipStream_t s_) : t(t_), role(role_), s(s_) {
    throw_on_error_(hkv_lock_begin(t, role, s));
  }
  ~RoleGuard() { (void)hkv_lock_end(t, role, s); }
};

}  // namespace detail

template <typename K, typename V, typename S = uint64_t, int Strategy = EvictStrategy::kLru,
          typename ArchTag = void>
class HashTable : public HashTableBase<K, V, S> {
 public:
  using size_type = size_t;
  using key_type = K;
  using value_type = V;
  using score_type = S;
  static constexpr int evict_strategy = Strategy;
  using allocator_type = BaseAllocator;

  static_assert(std::is_same<K, int64_t>::value || std::is_same<K, uint64_t>::value,
                "The key_type must be int64_t or uint64_t.");
  static_assert(std::is_same<S, uint64_t>::value || std::is_same<S, uint32_t>::value,
                "The score_type must be uint64_t or uint32_t.");
  /* merlin_hashtable.cuh:944-949 */
  static_assert(std::is_same<S, uint64_t>::value || Strategy == EvictStrategy::kCustomized,
                "The uint32_t score_type is only supported with EvictStrategy::kCustomized.");
  static_assert(std::is_trivially_copyable<V>::value, "value_type must be trivially copyable");
  static_assert(sizeof(size_type) == sizeof(uint64_t), "size_type must be 64 bits wide");

 public:
  HashTable() {}
  ~HashTable() {
    if (table_ != nullptr) {
      (void)hkv_table_destroy(table_);
      table_ = nullptr;
    }
    if (default_allocator_ && allocator_ != nullptr) delete allocator_;
  }

 private:
  HashTable(const HashTable&) = delete;
  HashTable& operator=(const HashTable&) = delete;
  HashTable(HashTable&&) = delete;
  HashTable& operator=(HashTable&&) = delete;

 public:
  void init(const HashTableOptions& options, allocator_type* allocator = nullptr) override {
    if (initialized_) return;
    options_ = options;
    hkv_options o;
    hkv_options_default(&o);
    o.init_capacity = options.init_capacity;
    o.max_capacity = options.max_capacity;
    o.max_hbm_for_vectors = options.max_hbm_for_vectors;
    o.max_bucket_size = options.max_bucket_size;
    o.dim = options.dim;
    o.max_load_factor = options.max_load_factor;
    o.block_size = options.block_size;
    o.io_block_size = options.io_block_size;
    o.device_id = options.device_id;
    o.io_by_cpu = options.io_by_cpu;
    o.use_constant_memory = options.use_constant_memory;
    o.reserved_key_start_bit = options.reserved_key_start_bit;
    o.num_of_buckets_per_alloc = options.num_of_buckets_per_alloc;
    o.api_lock = options.api_lock;
    o.table_mode = static_cast<int>(options.table_mode);
    o.evict_strategy = Strategy;
    o.value_kind = detail::value_kind_of<V>();
    o.value_size = sizeof(V);
    o.score_size = sizeof(uint64_t); /* the table's own width; 32-bit scores are widened at the calls */
    default_allocator_ = (allocator == nullptr);
    allocator_ = default_allocator_ ? nullptr : allocator;
    if (allocator_ != nullptr) {
      hkv_allocator a{allocator_, &detail::alloc_cb, &detail::free_cb};
      throw_on_error_(hkv_table_create_with_allocator(&o, &a, &table_));
    } else {
      throw_on_error_(hkv_table_create(&o, &table_));
    }
    if (options_.device_id < 0) HKV_HIP_CHECK(hipGetDevice(&options_.device_id));
    initialized_ = true;
  }

  void insert_or_assign(const size_type n, const key_type* keys, const value_type* values,
                        const score_type* scores = nullptr, hipStream_t stream = 0,
                        bool unique_key = true, bool ignore_evict_strategy = false) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    throw_on_error_(hkv_insert_or_assign(table_, n, u64(keys), values, sc.get(), stream, unique_key,
                                         ignore_evict_strategy));
  }

  void insert_and_evict(const size_type n, const key_type* keys, const value_type* values,
                        const score_type* scores, key_type* evicted_keys,
                        value_type* evicted_values, score_type* evicted_scores,
                        size_type* d_evicted_counter, hipStream_t stream = 0,
                        bool unique_key = true, bool ignore_evict_strategy = false) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    detail::ScoresOut<S> es(evicted_scores, n, stream);
    throw_on_error_(hkv_insert_and_evict(table_, n, u64(keys), values, sc.get(), u64(evicted_keys),
                                         evicted_values, es.get(),
                                         reinterpret_cast<uint64_t*>(d_evicted_counter), stream,
                                         unique_key, ignore_evict_strategy));
    es.finish();
  }

  size_type insert_and_evict(const size_type n, const key_type* keys, const value_type* values,
                             const score_type* scores, key_type* evicted_keys,
                             value_type* evicted_values, score_type* evicted_scores,
                             hipStream_t stream = 0, bool unique_key = true,
                             bool ignore_evict_strategy = false) override {
    uint64_t cnt = 0;
    detail::ScoresIn<S> sc(scores, n, stream);
    detail::ScoresOut<S> es(evicted_scores, n, stream);
    throw_on_error_(hkv_insert_and_evict_count(table_, n, u64(keys), values, sc.get(),
                                               u64(evicted_keys), evicted_values, es.get(),
                                               stream, unique_key, ignore_evict_strategy, &cnt));
    es.finish();
    if (!std::is_same<S, uint64_t>::value) HKV_HIP_CHECK(hipStreamSynchronize(stream));
    return static_cast<size_type>(cnt);
  }

  void accum_or_assign(const size_type n, const key_type* keys, const value_type* value_or_deltas,
                       const bool* accum_or_assigns, const score_type* scores = nullptr,
                       hipStream_t stream = 0, bool ignore_evict_strategy = false) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    throw_on_error_(hkv_accum_or_assign(table_, n, u64(keys), value_or_deltas,
                                        reinterpret_cast<const uint8_t*>(accum_or_assigns), sc.get(),
                                        stream, ignore_evict_strategy));
  }

  void find_or_insert(const size_type n, const key_type* keys, value_type* values,
                      score_type* scores = nullptr, hipStream_t stream = 0,
                      bool unique_key = true, bool ignore_evict_strategy = false) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    throw_on_error_(hkv_find_or_insert(table_, n, u64(keys), values, sc.get(), stream, unique_key,
                                       ignore_evict_strategy));
  }

  void find_or_insert(const size_type n, const key_type* keys, value_type** values, bool* founds,
                      score_type* scores = nullptr, hipStream_t stream = 0,
                      bool unique_key = true, bool ignore_evict_strategy = false,
                      key_type** locked_key_ptrs = nullptr) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    if (locked_key_ptrs != nullptr) {
      /* merlin_hashtable.cuh:1914-1918 */
      if (!unique_key)
        throw std::invalid_argument("unique_key should be true and max_bucket_size should be larger.");
      throw_on_error_(hkv_find_or_insert_ptr_lock(
          table_, n, u64(keys), reinterpret_cast<void**>(values), reinterpret_cast<uint8_t*>(founds),
          sc.get(), reinterpret_cast<uint64_t**>(locked_key_ptrs), stream, ignore_evict_strategy));
      return;
    }
    throw_on_error_(hkv_find_or_insert_ptr(table_, n, u64(keys), reinterpret_cast<void**>(values),
                                           reinterpret_cast<uint8_t*>(founds), sc.get(), stream,
                                           unique_key, ignore_evict_strategy));
  }

  /* merlin_hashtable.cuh:1982-2012 */
  void lock_keys(const size_type n, key_type const* keys, key_type** locked_key_ptrs,
                 bool* succeededs = nullptr, hipStream_t stream = 0,
                 score_type const* scores = nullptr) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    throw_on_error_(hkv_lock_keys(table_, n, u64(keys),
                                  reinterpret_cast<uint64_t**>(locked_key_ptrs),
                                  reinterpret_cast<uint8_t*>(succeededs), sc.get(), stream));
  }
  /* merlin_hashtable.cuh:2026-2044 */
  void unlock_keys(const size_type n, key_type** locked_key_ptrs, const key_type* keys,
                   bool* succeededs = nullptr, hipStream_t stream = 0) override {
    throw_on_error_(hkv_unlock_keys(table_, n, reinterpret_cast<uint64_t**>(locked_key_ptrs),
                                    u64(keys), reinterpret_cast<uint8_t*>(succeededs), stream));
  }

  void assign(const size_type n, const key_type* keys, const value_type* values,
              const score_type* scores = nullptr, hipStream_t stream = 0,
              bool unique_key = true) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    throw_on_error_(hkv_assign(table_, n, u64(keys), values, sc.get(), stream, unique_key));
  }
  void assign_scores(const size_type n, const key_type* keys, const score_type* scores = nullptr,
                     hipStream_t stream = 0, bool unique_key = true) override {
    detail::ScoresIn<S> sc(scores, n, stream);
    throw_on_error_(hkv_assign_scores(table_, n, u64(keys), sc.get(), stream, unique_key));
  }
  /* alias of assign_scores (merlin_hashtable.cuh:2285-2290) */
  void assign(const size_type n, const key_type* keys, const score_type* scores = nullptr,
              hipStream_t stream = 0, bool unique_key = true) override {
    assign_scores(n, keys, scores, stream, unique_key);
  }
  void assign_values(const size_type n, const key_type* keys, const value_type* values,
                     hipStream_t stream = 0, bool unique_key = true) override {
    throw_on_error_(hkv_assign_values(table_, n, u64(keys), values, stream, unique_key));
  }

  void find(const size_type n, const key_type* keys, value_type* values, bool* founds,
            score_type* scores = nullptr, hipStream_t stream = 0) const override {
    detail::ScoresOut<S> so(scores, n, stream);
    throw_on_error_(hkv_find(table_, n, u64(keys), values, reinterpret_cast<uint8_t*>(founds),
                             so.get(), stream));
    so.finish();
  }
  void find(const size_type n, const key_type* keys, value_type* values, key_type* missed_keys,
            int* missed_indices, int* missed_size, score_type* scores = nullptr,
            hipStream_t stream = 0) const override {
    detail::ScoresOut<S> so(scores, n, stream);
    throw_on_error_(hkv_find_missed(table_, n, u64(keys), values, u64(missed_keys), missed_indices,
                                    missed_size, so.get(), stream));
    so.finish();
  }
  void find(const size_type n, const key_type* keys, value_type** values, bool* founds,
            score_type* scores = nullptr, hipStream_t stream = 0,
            bool unique_key = true) const override {
    detail::ScoresOut<S> so(scores, n, stream);
    throw_on_error_(hkv_find_ptr(table_, n, u64(keys), reinterpret_cast<void**>(values),
                                 reinterpret_cast<uint8_t*>(founds), so.get(), stream, unique_key));
    so.finish();
  }
  /* merlin_hashtable.cuh:2811-2843 */
  void find_and_update(const size_type n, const key_type* keys, value_type** values, bool* founds,
                       score_type* scores = nullptr, hipStream_t stream = 0,
                       bool unique_key = true) override {
    if (!unique_key)
      throw std::runtime_error(
          "Not support update score when keys are not unique or bucket capacity is small.");
    detail::ScoresIn<S> sc(scores, n, stream);
    throw_on_error_(hkv_find_and_update(table_, n, u64(keys), reinterpret_cast<void**>(values),
                                        reinterpret_cast<uint8_t*>(founds),
                                        const_cast<uint64_t*>(sc.get()), stream));
  }
  void contains(const size_type n, const key_type* keys, bool* founds,
                hipStream_t stream = 0) const override {
    throw_on_error_(hkv_contains(table_, n, u64(keys), reinterpret_cast<uint8_t*>(founds), stream));
  }

  void erase(const size_type n, const key_type* keys, hipStream_t stream = 0) override {
    throw_on_error_(hkv_erase(table_, n, u64(keys), stream));
  }

  /* erase every entry for which pred(key, score, pattern, threshold) holds;
   * returns how many (merlin_hashtable.cuh:2963-2996).  Synchronises `stream`. */
  template <template <typename, typename> class PredFunctor>
  size_type erase_if(const key_type& pattern, const score_type& threshold, hipStream_t stream = 0) {
    detail::DeviceWord<unsigned long long> count(stream);
    unsigned long long* d_count = count.get();
    hipLaunchKernelGGL((hkv::zero_word_kernel<unsigned long long>), dim3(1), dim3(1), 0, stream,
                       d_count);
    {
      /* the role is taken first: it keeps other host threads from growing the table (which
       * frees the arenas the view points at) until this call has enqueued its kernel */
      detail::RoleGuard g(table_, 2, stream);
      hkv_table_view v;
      throw_on_error_(hkv_table_get_view(table_, &v));
      const unsigned blocks = hkv::scan_grid(v.capacity, 256);
      hipLaunchKernelGGL((hkv::erase_if_kernel<detail::PredAdapter<K, S, PredFunctor>>),
                         dim3(blocks), dim3(256), 0, stream, v,
                         detail::PredAdapter<K, S, PredFunctor>(), static_cast<uint64_t>(pattern),
                         static_cast<uint64_t>(threshold), d_count);
      HKV_HIP_CHECK(hipGetLastError());
    }
    return static_cast<size_type>(count.read());
  }

  /* merlin_hashtable.cuh:3008-3052: pred.template operator()<GroupSize>(key, value, score, tile)
   * decides; returns how many entries were erased.  Synchronises `stream`. */
  template <typename PredFunctor>
  size_type erase_if_v2(PredFunctor& pred, hipStream_t stream = 0) {
    detail::DeviceWord<unsigned long long> count(stream);
    unsigned long long* d_count = count.get();
    hipLaunchKernelGGL((hkv::zero_word_kernel<unsigned long long>), dim3(1), dim3(1), 0, stream,
                       d_count);
    {
      detail::RoleGuard g(table_, 2, stream);
      hkv_table_view v;
      throw_on_error_(hkv_table_get_view(table_, &v));
      const uint64_t n = v.capacity;
      const unsigned blocks = hkv::scan_grid(n, 128);
      const uint64_t dim = options_.dim;
      if (dim >= 32 && n % 32 == 0)
        hipLaunchKernelGGL((hkv::erase_if_v2_kernel<K, V, S, PredFunctor, 32>), dim3(blocks),
                           dim3(128), 0, stream, v, n, pred, d_count);
      else if (dim >= 16 && n % 16 == 0)
        hipLaunchKernelGGL((hkv::erase_if_v2_kernel<K, V, S, PredFunctor, 16>), dim3(blocks),
                           dim3(128), 0, stream, v, n, pred, d_count);
      else if (dim >= 8 && n % 8 == 0)
        hipLaunchKernelGGL((hkv::erase_if_v2_kernel<K, V, S, PredFunctor, 8>), dim3(blocks),
                           dim3(128), 0, stream, v, n, pred, d_count);
      else
        hipLaunchKernelGGL((hkv::erase_if_v2_kernel<K, V, S, PredFunctor, 1>), dim3(blocks),
                           dim3(128), 0, stream, v, n, pred, d_count);
      HKV_HIP_CHECK(hipGetLastError());
    }
    return static_cast<size_type>(count.read());
  }

  /* merlin_hashtable.cuh:3307-3348 */
  template <typename PredFunctor>
  void export_batch_if_v2(PredFunctor& pred, size_type n, const size_type offset,
                          size_type* d_counter, key_type* keys, value_type* values,
                          score_type* scores = nullptr, hipStream_t stream = 0) const {
    detail::RoleGuard g(table_, 0, stream);
    hkv_table_view v;
    throw_on_error_(hkv_table_get_view(table_, &v));
    hipLaunchKernelGGL((hkv::zero_word_kernel<size_type>), dim3(1), dim3(1), 0, stream, d_counter);
    if (offset >= v.capacity) return;
    n = std::min<size_type>(v.capacity - offset, n);
    if (n == 0) return;
    const unsigned blocks = hkv::export_grid(n, hkv::kExportV2Threads);
    const uint64_t dim = options_.dim;
    auto* cnt = reinterpret_cast<unsigned long long*>(d_counter);
    if (dim >= 32 && n % 32 == 0)
      hipLaunchKernelGGL((hkv::export_if_v2_kernel<K, V, S, PredFunctor, 32>), dim3(blocks),
                         dim3(128), 0, stream, v, n, offset, pred, cnt, keys, values, scores);
    else if (dim >= 16 && n % 16 == 0)
      hipLaunchKernelGGL((hkv::export_if_v2_kernel<K, V, S, PredFunctor, 16>), dim3(blocks),
                         dim3(128), 0, stream, v, n, offset, pred, cnt, keys, values, scores);
    else if (dim >= 8 && n % 8 == 0)
      hipLaunchKernelGGL((hkv::export_if_v2_kernel<K, V, S, PredFunctor, 8>), dim3(blocks),
                         dim3(128), 0, stream, v, n, offset, pred, cnt, keys, values, scores);
    else
      hipLaunchKernelGGL((hkv::export_if_v2_kernel<K, V, S, PredFunctor, 1>), dim3(blocks),
                         dim3(128), 0, stream, v, n, offset, pred, cnt, keys, values, scores);
    HKV_HIP_CHECK(hipGetLastError());
  }

  /* merlin_hashtable.cuh:3372-3412: f.template operator()<GroupSize>(key, value, score, tile)
   * is applied to every slot of [first, last), reserved keys included */
  template <typename ExecutionFunc>
  void for_each(const size_type first, const size_type last, ExecutionFunc& f,
                hipStream_t stream = 0) {
    detail::RoleGuard g(table_, 2, stream);
    hkv_table_view v;
    throw_on_error_(hkv_table_get_view(table_, &v));
    if (first >= v.capacity || last > v.capacity || first >= last) return;
    throw_on_error_(hkv_scores_changed(table_)); /* the functor may write scores */
    const uint64_t n = last - first;
    const unsigned blocks = static_cast<unsigned>(std::min<uint64_t>((n + 127) / 128, 16384));
    const uint64_t dim = options_.dim;
    if (dim >= 32 && n % 32 == 0)
      hipLaunchKernelGGL((hkv::traverse_kernel<K, V, S, ExecutionFunc, 32>), dim3(blocks), dim3(128),
                         0, stream, v, n, first, f);
    else if (dim >= 16 && n % 16 == 0)
      hipLaunchKernelGGL((hkv::traverse_kernel<K, V, S, ExecutionFunc, 16>), dim3(blocks), dim3(128),
                         0, stream, v, n, first, f);
    else if (dim >= 8 && n % 8 == 0)
      hipLaunchKernelGGL((hkv::traverse_kernel<K, V, S, ExecutionFunc, 8>), dim3(blocks), dim3(128),
                         0, stream, v, n, first, f);
    else
      hipLaunchKernelGGL((hkv::traverse_kernel<K, V, S, ExecutionFunc, 1>), dim3(blocks), dim3(128),
                         0, stream, v, n, first, f);
    HKV_HIP_CHECK(hipGetLastError());
  }

  void clear(hipStream_t stream = 0) override { throw_on_error_(hkv_clear(table_, stream)); }

  void export_batch(size_type n, const size_type offset, size_type* d_counter, key_type* keys,
                    value_type* values, score_type* scores = nullptr,
                    hipStream_t stream = 0) const override {
    detail::ScoresOut<S> so(scores, n, stream);
    throw_on_error_(hkv_export_batch(table_, n, offset, reinterpret_cast<uint64_t*>(d_counter),
                                     u64(keys), values, so.get(), stream));
    so.finish();
  }

  size_type export_batch(const size_type n, const size_type offset, key_type* keys,
                         value_type* values, score_type* scores = nullptr,
                         hipStream_t stream = 0) const override {
    detail::DeviceWord<size_type> count(stream);
    export_batch(n, offset, count.get(), keys, values, scores, stream);
    return count.read();
  }

  /* merlin_hashtable.cuh:3193-3276: the caller's device functor decides. */
  template <template <typename, typename> class PredFunctor>
  void export_batch_if(const key_type& pattern, const score_type& threshold, size_type n,
                       const size_type offset, size_type* d_counter, key_type* keys,
                       value_type* values, score_type* scores = nullptr,
                       hipStream_t stream = 0) const {
    detail::RoleGuard g(table_, 0, stream);
    hkv_table_view v;
    throw_on_error_(hkv_table_get_view(table_, &v));
    hipLaunchKernelGGL((hkv::zero_word_kernel<size_type>), dim3(1), dim3(1), 0, stream, d_counter);
    if (offset >= v.capacity) return;
    n = std::min<size_type>(v.capacity - offset, n);
    if (n == 0) return;
    detail::ScoresOut<S> so(scores, n, stream);
    const unsigned blocks = hkv::export_grid(n, hkv::kExportThreads);
    hipLaunchKernelGGL((hkv::export_if_kernel<detail::PredAdapter<K, S, PredFunctor>>),
                       dim3(blocks), dim3(256), 0, stream, v,
                       detail::PredAdapter<K, S, PredFunctor>(), static_cast<uint64_t>(pattern),
                       static_cast<uint64_t>(threshold), static_cast<uint64_t>(offset),
                       static_cast<uint64_t>(n), reinterpret_cast<unsigned long long*>(d_counter),
                       u64(keys), reinterpret_cast<uint8_t*>(values), so.get());
    HKV_HIP_CHECK(hipGetLastError());
    so.finish();
  }

  /* merlin_hashtable.cuh:3460-3476: the count goes to a device word, asynchronously */
  template <template <typename, typename> class PredFunctor>
  void size_if(const key_type& pattern, const score_type& threshold, size_type* d_counter,
               hipStream_t stream = 0) const {
    detail::RoleGuard g(table_, 0, stream);
    hkv_table_view v;
    throw_on_error_(hkv_table_get_view(table_, &v));
    hipLaunchKernelGGL((hkv::zero_word_kernel<size_type>), dim3(1), dim3(1), 0, stream, d_counter);
    const unsigned blocks = hkv::scan_grid(v.capacity, 256);
    hipLaunchKernelGGL((hkv::size_if_kernel<detail::PredAdapter<K, S, PredFunctor>>), dim3(blocks),
                       dim3(256), 0, stream, v, detail::PredAdapter<K, S, PredFunctor>(),
                       static_cast<uint64_t>(pattern), static_cast<uint64_t>(threshold),
                       reinterpret_cast<unsigned long long*>(d_counter));
    HKV_HIP_CHECK(hipGetLastError());
  }

  /* convenience form without a counter argument (not in the reference): returns the count and
   * synchronises `stream` */
  template <template <typename, typename> class PredFunctor>
  size_type size_if(const key_type& pattern, const score_type& threshold,
                    hipStream_t stream = 0) const {
    detail::DeviceWord<size_type> count(stream);
    size_if<PredFunctor>(pattern, threshold, count.get(), stream);
    return count.read();
  }

  bool empty(hipStream_t stream = 0) const override { return size(stream) == 0; }

  size_type size(hipStream_t stream = 0) const override {
    uint64_t n = 0;
    throw_on_error_(hkv_size(table_, stream, &n));
    return static_cast<size_type>(n);
  }

  size_type capacity() const override { return hkv_capacity(table_); }

  /* merlin_hashtable.cuh:3503-3541 */
  void reserve(const size_type new_capacity, hipStream_t stream = 0) override {
    throw_on_error_(hkv_reserve(table_, new_capacity, stream));
  }

  float load_factor(hipStream_t stream = 0) const override {
    float lf = 0.f;
    throw_on_error_(hkv_load_factor(table_, stream, &lf));
    return lf;
  }

  /* merlin_hashtable.cuh:3561-3574 */
  void set_max_capacity(size_type new_max_capacity) override {
    if (new_max_capacity == 0 || (new_max_capacity & (new_max_capacity - 1)) != 0)
      throw std::invalid_argument("None power-of-2 new_max_capacity is not supported.");
    throw_on_error_(hkv_set_max_capacity(table_, new_max_capacity));
    if (new_max_capacity >= capacity()) options_.max_capacity = new_max_capacity;
  }

  size_type dim() const noexcept override { return options_.dim; }
  size_type max_bucket_size() const noexcept override { return options_.max_bucket_size; }
  size_type bucket_count() const noexcept override { return hkv_bucket_count(table_); }

  /*
   * save / load, merlin_hashtable.cuh:3615-3758: the table is exported in
   * windows of the slot range that fit the workspace, staged through pinned
   * host memory, and handed to the file; load inserts with the saved scores
   * (ignore_evict_strategy).
   */
  size_type save(BaseKVFile<K, V, S>* file, const size_t max_workspace_size = 1L * 1024 * 1024,
                 hipStream_t stream = 0) const override {
    const size_type tuple_size = sizeof(K) + sizeof(S) + sizeof(V) * dim();
    MERLIN_CHECK(max_workspace_size >= tuple_size,
                 "[HierarchicalKV] max_workspace_size is smaller than a single `key + score + value` tuple! Please set a larger value!");
    const size_type total = capacity();
    const size_type window = std::max<size_type>(max_workspace_size / tuple_size, 1);
    /* released on every way out, also when export_batch or the file throws */
    detail::StageBuffer<K> dk(window, false), hk(window, true);
    detail::StageBuffer<V> dv(window * dim(), false), hv(window * dim(), true);
    detail::StageBuffer<S> ds(window, false), hs(window, true);
    K *d_keys = dk.get(), *h_keys = hk.get();
    V *d_vals = dv.get(), *h_vals = hv.get();
    S *d_scores = ds.get(), *h_scores = hs.get();
    size_type written = 0;
    for (size_type off = 0; off < total; off += window) {
      const size_type c = export_batch(window, off, d_keys, d_vals, d_scores, stream);
      if (c == 0) continue;
      HKV_HIP_CHECK(hipMemcpyAsync(h_keys, d_keys, c * sizeof(K), hipMemcpyDeviceToHost, stream));
      HKV_HIP_CHECK(hipMemcpyAsync(h_vals, d_vals, c * sizeof(V) * dim(), hipMemcpyDeviceToHost, stream));
      HKV_HIP_CHECK(hipMemcpyAsync(h_scores, d_scores, c * sizeof(S), hipMemcpyDeviceToHost, stream));
      HKV_HIP_CHECK(hipStreamSynchronize(stream));
      written += file->write(c, dim(), h_keys, h_vals, h_scores);
    }
    return written;
  }

  size_type load(BaseKVFile<K, V, S>* file, const size_t max_workspace_size = 1L * 1024 * 1024,
                 hipStream_t stream = 0) override {
    const size_type tuple_size = sizeof(K) + sizeof(S) + sizeof(V) * dim();
    MERLIN_CHECK(max_workspace_size >= tuple_size,
                 "[HierarchicalKV] max_workspace_size is smaller than a single `key + score + value` tuple! Please set a larger value!");
    const size_type window = std::max<size_type>(max_workspace_size / tuple_size, 1);
    /* released on every way out, also when export_batch or the file throws */
    detail::StageBuffer<K> dk(window, false), hk(window, true);
    detail::StageBuffer<V> dv(window * dim(), false), hv(window * dim(), true);
    detail::StageBuffer<S> ds(window, false), hs(window, true);
    K *d_keys = dk.get(), *h_keys = hk.get();
    V *d_vals = dv.get(), *h_vals = hv.get();
    S *d_scores = ds.get(), *h_scores = hs.get();
    size_type loaded = 0;
    while (true) {
      const size_type c = file->read(window, dim(), h_keys, h_vals, h_scores);
      if (c == 0) break;
      HKV_HIP_CHECK(hipMemcpyAsync(d_keys, h_keys, c * sizeof(K), hipMemcpyHostToDevice, stream));
      HKV_HIP_CHECK(hipMemcpyAsync(d_vals, h_vals, c * sizeof(V) * dim(), hipMemcpyHostToDevice, stream));
      HKV_HIP_CHECK(hipMemcpyAsync(d_scores, h_scores, c * sizeof(S), hipMemcpyHostToDevice, stream));
      insert_or_assign(c, d_keys, d_vals, d_scores, stream, true, true);
      HKV_HIP_CHECK(hipStreamSynchronize(stream));
      loaded += c;
    }
    return loaded;
  }

  void set_global_epoch(const uint64_t epoch) override {
    throw_on_error_(hkv_set_global_epoch(table_, epoch));
  }

  /* this build's additions */
  bool is_pure_hbm() const { return hkv_is_pure_hbm(table_) != 0; }
  hkv_table* native_handle() const { return table_; }

 private:
  static const uint64_t* u64(const K* p) { return reinterpret_cast<const uint64_t*>(p); }
  static uint64_t* u64(K* p) { return reinterpret_cast<uint64_t*>(p); }

  HashTableOptions options_;
  hkv_table* table_ = nullptr;
  bool initialized_ = false;
  allocator_type* allocator_ = nullptr;
  bool default_allocator_ = true;
};

}  // namespace merlin
}  // namespace nv

#endif  // MERLIN_HASHTABLE_HPP_
