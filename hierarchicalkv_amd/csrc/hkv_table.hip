/*
 * Host side of the table and the C ABI (include/hkv_c_api.h).
 *
 * What lives here: argument checks with the reference's messages
 * (merlin_hashtable.cuh:1016-1048, 3832-3861), table memory (flat arenas; HBM
 * first, pinned mapped host memory for value rows past max_hbm_for_vectors),
 * the stream-ordered group lock, and the choice of kernel instance per call.
 */
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <algorithm>
#include <atomic>
#include <condition_variable>
#include <cstdarg>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <map>
#include <mutex>
#include <new>
#include <string>
#include <thread>
#include <vector>

#include "hkv_c_api.h"
#include "hkv_misc.hpp"
#include "hkv_upsert.hpp"
#include "hkv_dedup.hpp"
#include "hkv_dual.hpp"
#include "hkv_grouped.hpp"
#include "hkv_keylocks.hpp"

using namespace hkv;

namespace {

thread_local std::string g_err;

int fail(int code, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof buf, fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

#define HKV_HIP(expr)                                                        \
  do {                                                                       \
    hipError_t e_ = (expr);                                                  \
    if (e_ != hipSuccess)                                                    \
      return fail(HKV_ERROR_HIP, "%s:%d %s: %s", __FILE__, __LINE__, #expr,  \
                  hipGetErrorString(e_));                                    \
  } while (0)

#define HKV_TRY(expr)              \
  do {                             \
    int rc_ = (expr);              \
    if (rc_ != HKV_SUCCESS) return rc_; \
  } while (0)

bool ispow2(uint64_t x) { return x && !(x & (x - 1)); }

/*
 * Group lock with the three roles of group_shared_mutex (group_lock.cuh:43-56):
 * readers run with readers, updaters with updaters, an inserter runs alone.
 * The reference blocks the host on a one-thread kernel per call; here the
 * exclusion is expressed between streams with events, so a call never waits on
 * the host: begin() makes `stream` wait for the conflicting work already
 * enqueued on other streams, end() publishes what the call has just enqueued.
 *
 * A stream is only ever touched inside a call that was made on it (the caller
 * may destroy it right afterwards).  While the table has seen one stream, the
 * stream's own order is all that is needed and nothing is recorded.  When a
 * second stream turns up, the device is synchronised once (the first stream may
 * be gone by then); from then on every call records one event on its own
 * stream in end(), and begin() waits for the events of the conflicting roles.
 * Entries whose event has completed are dropped, so streams that come and go
 * leave nothing behind.
 */
class StreamGroupLock {
 public:
  enum Role { kReader = 0, kUpdater = 1, kInserter = 2 };

  ~StreamGroupLock() {
    for (auto& r : roles_)
      for (auto& kv : r) (void)hipEventDestroy(kv.second);
    for (hipEvent_t e : spare_) (void)hipEventDestroy(e);
  }

  hipError_t begin(Role role, hipStream_t s) {
    mu_.lock();
    hipError_t e = hipSuccess;
    if (!multi_) {
      if (!seen_one_) {
        seen_one_ = true;
        only_ = s;
      } else if (s != only_) {
        /* everything the first stream carries is complete after this, whether or not the
         * stream still exists */
        e = hipDeviceSynchronize();
        multi_ = true;
      }
    } else {
      for (int other = 0; other < 3 && e == hipSuccess; other++) {
        const bool clash = conflicts(role, (Role)other);
        for (auto it = roles_[other].begin(); it != roles_[other].end() && e == hipSuccess;) {
          if (hipEventQuery(it->second) == hipSuccess) { /* done: nobody needs to wait for it */
            spare_.push_back(it->second);
            it = roles_[other].erase(it);
            continue;
          }
          if (clash && it->first != s) e = hipStreamWaitEvent(s, it->second, 0);
          ++it;
        }
      }
    }
    if (e != hipSuccess) mu_.unlock();
    return e;
  }

  hipError_t end(Role role, hipStream_t s) {
    hipError_t e = hipSuccess;
    if (multi_) {
      auto it = roles_[role].find(s);
      if (it == roles_[role].end()) {
        hipEvent_t ev = nullptr;
        if (!spare_.empty()) {
          ev = spare_.back();
          spare_.pop_back();
        } else {
          e = hipEventCreateWithFlags(&ev, hipEventDisableTiming);
        }
        if (e == hipSuccess) it = roles_[role].emplace(s, ev).first;
      }
      if (e == hipSuccess) e = hipEventRecord(it->second, s);
    }
    mu_.unlock();
    return e;
  }

 private:
  /* Updaters on different streams are ordered among themselves as well (the reference
   * lets them overlap and pays a slot lock per key for it): an updater that is alone on
   * the table needs no slot locks. */
  static bool conflicts(Role a, Role b) {
    if (a == kInserter || b == kInserter) return true;
    if (a == kUpdater && b == kUpdater) return true;
    return a != b;
  }
  std::mutex mu_;
  bool seen_one_ = false, multi_ = false;
  hipStream_t only_ = nullptr;
  std::map<hipStream_t, hipEvent_t> roles_[3]; /* last event of each stream in each role */
  std::vector<hipEvent_t> spare_;
};

}  // namespace

struct hkv_table {
  hkv_options opts;
  View view;
  int device;
  bool pure_hbm;
  bool own_alloc;
  hkv_allocator alloc;
  void* d_meta;          /* digests + keys + scores + sizes + score bounds in one arena */
  std::atomic<uint64_t> keys_offered{0}; /* keys handed to upserts since creation or clear: above the size */
  bool score_bounds;     /* upserts into full buckets search victims through the score bounds
                            (HKV_SCORE_BOUNDS=0: off; switched off for good once a score-writing call
                            has been recorded into a HIP graph, see writes_scores_outside_bounds) */
  std::atomic<bool> bounds_stale{true}; /* a call may have written scores below the bounds */
  uint64_t bounds_epoch = 0; /* EpochLRU: epoch and era (clock >> 52: the low half of such a score */
  uint64_t bounds_era = 0;   /* wraps once per era) of the last call that used the bounds */
  uint64_t meta_bytes;
  void* d_values;        /* value rows in HBM */
  void* h_values;        /* host address of the pinned value rows (hybrid) */
  unsigned long long* d_counters; /* scratch words for size / size_if / the count-returning
                                     insert_and_evict: one per call in flight (CounterLease) */
  mutable std::mutex counter_mu;
  mutable std::condition_variable counter_cv;
  mutable std::vector<unsigned> counter_free;
  uint64_t epoch;
  Clock clock;
  mutable StreamGroupLock lock;
  bool reach_max_capacity; /* merlin_hashtable.cuh:1064: no further growth */
  bool keys_may_be_locked; /* LOCKED key words may sit in the table (lock_keys, the pointer
                              overload with locked_key_ptrs), until the count below reads 0 */
  bool locked_recount;     /* unlock_keys has run since the count was last read */
  unsigned long long* d_bound_caps; /* two device words: clock readings of the last calls that used the score bounds, used in turn */
  unsigned bound_cap_turn = 0;
  unsigned long long* d_score_floor; /* two device words, used in turn: the lowest score of a batch (score_floor_kernel) */
  unsigned score_floor_turn = 0;
  unsigned long long* d_bound_ceil;  /* device word: no bound of the table is above it (strategies with scores from the caller) */
  unsigned long long* d_load_sample; /* device word: the sum fast_load_factor reads back */
  unsigned long long* d_locked; /* device words (kLockedShards of them): slots left LOCKED by those calls, less the unlocked */
  bool dual;               /* TableMode::kMemory: two candidate buckets per key */
  bool io_by_cpu;          /* value rows of the writers are moved by host threads */
  std::mutex io_mutex;     /* one CPU-IO call at a time uses the staging area */
  void* io_stage;          /* pinned staging area of the CPU-IO calls, grown on demand */
  uint64_t io_stage_bytes;
};

namespace {

int table_alloc(hkv_table* t, int type, void** p, size_t bytes) {
  if (!t->own_alloc) {
    if (t->alloc.alloc(t->alloc.ctx, type, p, bytes) != 0 || !*p)
      return fail(HKV_ERROR_RUNTIME, "allocator failed for %zu bytes (type %d)", bytes, type);
    /* the kernels address the arenas in 16-byte units and 128-byte lines */
    if (((uintptr_t)*p & 255) != 0) {
      t->alloc.free(t->alloc.ctx, type, *p);
      *p = nullptr;
      return fail(HKV_ERROR_ARGUMENT, "the allocator must return memory aligned to 256 bytes");
    }
    return HKV_SUCCESS;
  }
  if (type == 0) {
    HKV_HIP(hipMalloc(p, bytes));
  } else {
    HKV_HIP(hipHostMalloc(p, bytes, hipHostMallocMapped | hipHostMallocPortable));
  }
  return HKV_SUCCESS;
}

void table_free(hkv_table* t, int type, void* p) {
  if (!p) return;
  if (!t->own_alloc) {
    t->alloc.free(t->alloc.ctx, type, p);
  } else if (type == 0) {
    (void)hipFree(p);
  } else {
    (void)hipHostFree(p);
  }
}

struct DeviceGuard {
  int prev = -1;
  bool ok = true;
  explicit DeviceGuard(int dev) {
    if (hipGetDevice(&prev) != hipSuccess) ok = false;
    if (ok && prev != dev && hipSetDevice(dev) != hipSuccess) ok = false;
  }
  ~DeviceGuard() {
    if (prev >= 0) (void)hipSetDevice(prev);
  }
};

struct LockGuard {
  const hkv_table* t;
  StreamGroupLock::Role role;
  hipStream_t s;
  bool held = false;
  LockGuard(const hkv_table* t_, StreamGroupLock::Role r, hipStream_t s_)
      : t(t_), role(r), s(s_) {}
  hipError_t acquire() {
    if (!t->opts.api_lock) return hipSuccess;
    hipError_t e = t->lock.begin(role, s);
    held = e == hipSuccess;
    return e;
  }
  ~LockGuard() {
    if (held) (void)t->lock.end(role, s);
  }
};

/* check_evict_strategy, merlin_hashtable.cuh:3832-3861 */
int check_scores_arg(const hkv_table* t, int strategy, const uint64_t* scores) {
  if ((strategy == HKV_LRU || strategy == HKV_EPOCH_LRU) && scores)
    return fail(HKV_ERROR_CHECK,
                "the scores should not be specified when running on LRU or Epoch LRU mode.");
  if ((strategy == HKV_LFU || strategy == HKV_EPOCH_LFU) && !scores)
    return fail(HKV_ERROR_CHECK,
                "the scores should be specified when running on LFU or Epoch LFU mode.");
  if (strategy == HKV_CUSTOMIZED && !scores)
    return fail(HKV_ERROR_CHECK,
                "the scores should be specified when running on customized mode.");
  if ((strategy == HKV_EPOCH_LRU || strategy == HKV_EPOCH_LFU) &&
      t->epoch == kIgnoredEpoch)
    return fail(HKV_ERROR_CHECK,
                "the global_epoch is invalid and should be assigned by calling "
                "`set_global_epoch` when running on Epoch LRU or Epoch LFU mode.");
  return HKV_SUCCESS;
}

/* widest unit (16, 4 or 1 bytes) that the row size and every pointer allow */
int pick_vec(uint32_t value_bytes, std::initializer_list<const void*> ptrs) {
  uintptr_t mis = value_bytes;
  for (const void* p : ptrs) mis |= (uintptr_t)p;
  if ((mis & 15) == 0) return 16;
  if ((mis & 3) == 0) return 4;
  return 1;
}

inline unsigned grid_for(uint64_t n) { return (unsigned)((n + kWave - 1) / kWave); }

/* units per lane that the bulk copy keeps in registers: rows of up to 8 * UPL
 * units go through in one pass (16-byte units: 128, 256, 512, 1024 bytes) */
int pick_upl(uint32_t value_bytes, int vec) {
  if (vec != 16) return 8;
  const uint32_t units = value_bytes / 16;
  if (units <= 8) return 1;
  if (units <= 16) return 2;
  if (units <= 32) return 4;
  return 8;
}

/* accum_or_assign adds element by element, so its unit must hold whole elements: the widest of
 * 16, 8, 4, 2 and 1 bytes that the row size and the pointer allow, or 0 when that is less than
 * one element (an odd address for 16-bit elements, and the like). */
int accum_unit(uint32_t value_bytes, const void* p, int kind) {
  const uint32_t elem[] = {1, 4, 8, 4, 8, 1, 2};
  const uintptr_t mis = value_bytes | (uintptr_t)p;
  int unit = 1;
  for (int u : {16, 8, 4, 2})
    if ((mis & (uintptr_t)(u - 1)) == 0) {
      unit = u;
      break;
    }
  return unit >= (int)elem[kind] ? unit : 0;
}

/* hkv_time_next_kernel: the pair of events that the calling thread's next main kernel (the one
 * kernel of a find or of an upsert-family call) is launched with.  The runtime stamps them with
 * the start and the end of that kernel's execution, so the time between them is the kernel's own,
 * without the gaps between the launches of a stream that events recorded around a call include. */
thread_local hipEvent_t g_time_start = nullptr, g_time_stop = nullptr;

template <class... KArgs, class... Args>
void launch_main(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t s, Args... args) {
  if (g_time_start) {
    hipExtLaunchKernelGGL(kernel, grid, block, 0, s, g_time_start, g_time_stop, 0, args...);
    g_time_start = g_time_stop = nullptr;
  } else {
    hipLaunchKernelGGL(kernel, grid, block, 0, s, args...);
  }
}

/* BOUNDS: the victim search reads the bucket's score bounds and one or two of its score lines
 * instead of all eight (hkv_upsert.hpp); for 16-byte units, which is what tables with rows of a
 * multiple of 16 bytes use. */
template <int OP, bool LOCKED_RULE, bool BOUNDS = false, int WAVES = 1, bool HOLD = false>
void launch_upsert(int vec, const View& v, const UpsertArgs& a, hipStream_t s) {
  const dim3 grid(grid_for((a.n + WAVES - 1) / WAVES)), block(kWave * WAVES);
  if constexpr (OP == kOpAccumOrAssign && !BOUNDS) {
    /* the two units that only the element-wise add needs */
    if (vec == 8) {
      launch_main(upsert_kernel<OP, 8, 8, LOCKED_RULE, false, WAVES, HOLD>, grid, block, s, v, a);
      return;
    }
    if (vec == 2) {
      launch_main(upsert_kernel<OP, 2, 8, LOCKED_RULE, false, WAVES, HOLD>, grid, block, s, v, a);
      return;
    }
  }
  if (OP == kOpFindOrInsertPtr) {
    launch_main(upsert_kernel<OP, 16, 1, LOCKED_RULE, BOUNDS, WAVES, HOLD>, grid, block, s, v, a);
    return;
  }
  if (vec == 16) {
    switch (pick_upl(v.value_bytes, 16)) {
      case 1: launch_main(upsert_kernel<OP, 16, 1, LOCKED_RULE, BOUNDS, WAVES, HOLD>, grid, block, s, v, a); break;
      case 2: launch_main(upsert_kernel<OP, 16, 2, LOCKED_RULE, BOUNDS, WAVES, HOLD>, grid, block, s, v, a); break;
      case 4: launch_main(upsert_kernel<OP, 16, 4, LOCKED_RULE, BOUNDS, WAVES, HOLD>, grid, block, s, v, a); break;
      default: launch_main(upsert_kernel<OP, 16, 8, LOCKED_RULE, BOUNDS, WAVES, HOLD>, grid, block, s, v, a); break;
    }
  } else if constexpr (!BOUNDS) {
    if (vec == 4)
      launch_main(upsert_kernel<OP, 4, 8, LOCKED_RULE, false, WAVES, HOLD>, grid, block, s, v, a);
    else
      launch_main(upsert_kernel<OP, 1, 8, LOCKED_RULE, false, WAVES, HOLD>, grid, block, s, v, a);
  }
}

/* insert_and_evict with `pair`: two wavefronts per workgroup share the claims on the
 * evicted-keys output (hkv_upsert.hpp) */
template <int OP, bool LOCKED_RULE, bool BOUNDS = false>
void launch_upsert_for(bool pair, int vec, const View& v, const UpsertArgs& a, hipStream_t s) {
  if constexpr (OP == kOpInsertOrAssign || OP == kOpFindOrInsert) {
    /* hybrid mode: the list of slots that stay LOCKED to the end of the launch */
    if (a.held_scores) {
      launch_upsert<OP, LOCKED_RULE, BOUNDS, 1, true>(vec, v, a, s);
      return;
    }
  }
  if constexpr (OP == kOpInsertAndEvict) {
    if (pair) {
      launch_upsert<OP, LOCKED_RULE, BOUNDS, 2>(vec, v, a, s);
      return;
    }
  }
  launch_upsert<OP, LOCKED_RULE, BOUNDS, 1>(vec, v, a, s);
}

/* The two kernels of the two-phase insert_or_assign (hkv_grouped.hpp) for a row size. */
template <template <int, int> class Launcher, class... Args>
void dispatch_vec_upl(int vec, uint32_t value_bytes, Args&&... args) {
  if (vec == 16) {
    switch (pick_upl(value_bytes, 16)) {
      case 1: Launcher<16, 1>::go(args...); break;
      case 2: Launcher<16, 2>::go(args...); break;
      case 4: Launcher<16, 4>::go(args...); break;
      default: Launcher<16, 8>::go(args...); break;
    }
  } else if (vec == 4) {
    Launcher<4, 8>::go(args...);
  } else {
    Launcher<1, 8>::go(args...);
  }
}

template <int VEC, int UPL>
struct LaunchHits {
  static void go(const View& v, const UpsertArgs& a, const ChainArgs& c, hipStream_t s) {
    hipLaunchKernelGGL((upsert_hits_kernel<VEC>), dim3(grid_for(a.n)), dim3(kWave), 0, s, v, a, c);
  }
};
template <int VEC, int UPL>
struct LaunchMisses {
  static void go(const View& v, const UpsertArgs& a, const ChainArgs& c, hipStream_t s) {
    hipLaunchKernelGGL((chained_miss_kernel<VEC, UPL>), dim3(grid_for(v.buckets_num)), dim3(kWave), 0,
                       s, v, a, c);
  }
};

/* ---- the two-phase insert_or_assign on a scratch area that is part of the library image -------
 * hkv_insert_or_assign_noalloc: list heads and links live in a file-scope device array, so the
 * call allocates nothing.  In host code the array's name is only a handle for
 * the symbol: its device address is looked up once per device (each device holds its own copy
 * of the array) and that pointer is what the kernels and the clearing launch get. */
constexpr uint64_t kNoAllocMaxBuckets = UINT64_C(1) << 20; /* capacity up to 2^27 */
constexpr uint64_t kNoAllocMaxKeys = UINT64_C(1) << 20;

}  // namespace
static __device__ __align__(256) uint32_t g_noalloc_scratch[kNoAllocMaxBuckets + kNoAllocMaxKeys];
namespace {

constexpr int kMaxDevices = 64;
std::mutex g_noalloc_mu;
uint32_t* g_noalloc_ptr[kMaxDevices]; /* device address of g_noalloc_scratch, per device */

/* The device's copy of the scratch array.  The caller has made `device` current. */
int noalloc_scratch(int device, uint32_t** out) {
  if (device < 0 || device >= kMaxDevices)
    return fail(HKV_ERROR_UNSUPPORTED, "device %d: the scratch table holds %d devices", device, kMaxDevices);
  std::lock_guard<std::mutex> g(g_noalloc_mu);
  if (!g_noalloc_ptr[device]) {
    void* p = nullptr;
    HKV_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(g_noalloc_scratch)));
    if (!p) return fail(HKV_ERROR_HIP, "hipGetSymbolAddress returned a null address");
    g_noalloc_ptr[device] = (uint32_t*)p;
  }
  *out = g_noalloc_ptr[device];
  return HKV_SUCCESS;
}

constexpr unsigned kCounterWords = 128;
/* behind the counters: d_bound_caps[2], d_score_floor[2], d_bound_ceil, d_load_sample, two spare
 * words, then d_locked (kLockedShards words, a 128-byte line apart) */
constexpr unsigned kExtraWords = 8 + kLockedShards * kLockedStride;

/* A device word for a call that returns a count.  The word belongs to the call from the
 * lease to its end (the call zeroes it on its stream, a kernel adds to it, the host reads it
 * back after a stream synchronisation), so host threads inside such calls never share one;
 * when all words are out, the next caller waits for one to come back. */
class CounterLease {
 public:
  CounterLease(const hkv_table* t, hipStream_t s) : t_(t), s_(s) {
    std::unique_lock<std::mutex> g(t->counter_mu);
    t->counter_cv.wait(g, [&] { return !t->counter_free.empty(); });
    idx_ = t->counter_free.back();
    t->counter_free.pop_back();
  }
  ~CounterLease() {
    /* an early return may have left work on the stream that still writes the word */
    if (!read_) (void)hipStreamSynchronize(s_);
    {
      std::lock_guard<std::mutex> g(t_->counter_mu);
      t_->counter_free.push_back(idx_);
    }
    t_->counter_cv.notify_one();
  }
  CounterLease(const CounterLease&) = delete;
  CounterLease& operator=(const CounterLease&) = delete;
  unsigned long long* word() const { return t_->d_counters + idx_; }
  /* the word's value once everything enqueued on the stream so far has run */
  int read(uint64_t* out) {
    unsigned long long h = 0;
    HKV_HIP(hipMemcpyAsync(&h, word(), sizeof h, hipMemcpyDeviceToHost, s_));
    HKV_HIP(hipStreamSynchronize(s_));
    read_ = true;
    *out = h;
    return HKV_SUCCESS;
  }

 private:
  const hkv_table* t_;
  hipStream_t s_;
  unsigned idx_ = 0;
  bool read_ = false;
};

/* Ties the device counter to the host's CLOCK_REALTIME: the best of a few samples (shortest
 * host interval around the launch) gives the epoch time of tick 0. */
int sync_clock(hkv_table* t) {
  auto host_ns = []() {
    struct timespec ts;
    clock_gettime(CLOCK_REALTIME, &ts);
    return (uint64_t)ts.tv_sec * UINT64_C(1000000000) + (uint64_t)ts.tv_nsec;
  };
  unsigned long long* d = t->d_counters;
  uint64_t best_span = ~UINT64_C(0);
  for (int rep = 0; rep < 4; rep++) {
    const uint64_t t0 = host_ns();
    hipLaunchKernelGGL(clock_sample_kernel, dim3(1), dim3(1), 0, 0, d);
    HKV_HIP(hipGetLastError());
    HKV_HIP(hipDeviceSynchronize());
    const uint64_t t1 = host_ns();
    unsigned long long ticks = 0;
    HKV_HIP(hipMemcpy(&ticks, d, sizeof ticks, hipMemcpyDeviceToHost));
    if (t1 - t0 < best_span) {
      best_span = t1 - t0;
      t->clock.offset = t0 + (t1 - t0) / 2 - (uint64_t)ticks * t->clock.ns_per_tick;
    }
  }
  HKV_HIP(hipMemset(d, 0, (kCounterWords + kExtraWords) * sizeof(unsigned long long)));
  return HKV_SUCCESS;
}

/* The memory of one table geometry. */
struct TableMem {
  void* d_meta;
  uint64_t meta_bytes;
  void* d_values;
  void* h_values;
};

void free_arenas(hkv_table* t, TableMem& m) {
  table_free(t, 0, m.d_meta);
  table_free(t, 0, m.d_values);
  table_free(t, 1, m.h_values);
  m = TableMem{};
}

/* Arenas for `buckets_num` buckets, filled with EMPTY: the geometry fields of
 * `v` (everything that does not depend on the bucket count is taken as is).
 * On failure the caller frees what `m` holds. */
int alloc_arenas(hkv_table* t, uint64_t buckets_num, View& v, TableMem& m) {
  v.buckets_num = buckets_num;
  v.capacity = buckets_num * kBucketSize;
  v.pow2_buckets = ispow2(buckets_num);
  /* metadata arena: digests | keys | scores | sizes (dual-bucket tables) | score bounds, each 256-byte aligned */
  auto up = [](uint64_t x) { return (x + 255) & ~UINT64_C(255); };
  const uint64_t off_keys = up(v.capacity);
  const uint64_t off_scores = off_keys + up(v.capacity * 8);
  const uint64_t off_sizes = off_scores + up(v.capacity * 8);
  const uint64_t off_bounds = off_sizes + (t->dual ? up(v.buckets_num * 4) : 0);
  m.meta_bytes = off_bounds + (t->score_bounds ? up(v.buckets_num * 8 * sizeof(uint64_t)) : 0);
  HKV_TRY(table_alloc(t, 0, &m.d_meta, m.meta_bytes));
  uint8_t* base = (uint8_t*)m.d_meta;
  v.digests = base;
  v.keys = (uint64_t*)(base + off_keys);
  v.scores = (uint64_t*)(base + off_scores);
  /* keys per bucket: only the two-choice placement of a dual-bucket table reads them */
  v.sizes = t->dual ? (int32_t*)(base + off_sizes) : nullptr;
  v.bounds = t->score_bounds ? (uint64_t*)(base + off_bounds) : nullptr;
  /* value rows: whole buckets in HBM while max_hbm_for_vectors lasts
   * (initialize_buckets, core_kernels.cuh:195-236), the rest pinned + mapped */
  const uint64_t bucket_bytes = (uint64_t)kBucketSize * v.value_bytes;
  /* a dual-bucket table must be created with max_hbm_for_vectors == 0 and is meant to be
   * all-HBM (merlin_hashtable.cuh:1000-1002): its rows go to HBM */
  const uint64_t hbm_buckets =
      t->dual ? v.buckets_num
              : std::min<uint64_t>(v.buckets_num, t->opts.max_hbm_for_vectors / bucket_bytes);
  v.hbm_slots = hbm_buckets * kBucketSize;
  v.values = nullptr;
  v.host_values = nullptr;
  if (hbm_buckets) {
    HKV_TRY(table_alloc(t, 0, &m.d_values, hbm_buckets * bucket_bytes));
    v.values = (uint8_t*)m.d_values;
  }
  if (hbm_buckets != v.buckets_num) {
    HKV_TRY(table_alloc(t, 1, &m.h_values, (v.buckets_num - hbm_buckets) * bucket_bytes));
    void* dp = nullptr;
    hipError_t e = hipHostGetDevicePointer(&dp, m.h_values, 0);
    if (e != hipSuccess)
      return fail(HKV_ERROR_HIP, "hipHostGetDevicePointer: %s", hipGetErrorString(e));
    v.host_values = (uint8_t*)dp;
  }
  const uint64_t groups = v.capacity / 16;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, 0, v, 1);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipDeviceSynchronize();
  if (e != hipSuccess) return fail(HKV_ERROR_HIP, "table fill: %s", hipGetErrorString(e));
  return HKV_SUCCESS;
}

/* One doubling: new arenas, rehash, swap.  Caller holds the inserter role and
 * the device is idle. */
int double_table(hkv_table* t, hipStream_t s) {
  View nv = t->view;
  TableMem mem{};
  int rc = alloc_arenas(t, t->view.buckets_num * 2, nv, mem);
  if (rc) {
    free_arenas(t, mem);
    return rc;
  }
  const uint64_t waves = t->view.capacity / kWave;
  hipLaunchKernelGGL(rehash_kernel, dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, s, t->view, nv);
  hipError_t e = hipGetLastError();
  if (e == hipSuccess) e = hipDeviceSynchronize();
  if (e != hipSuccess) {
    free_arenas(t, mem);
    return fail(HKV_ERROR_HIP, "rehash: %s", hipGetErrorString(e));
  }
  TableMem old{t->d_meta, t->meta_bytes, t->d_values, t->h_values};
  t->d_meta = mem.d_meta;
  t->meta_bytes = mem.meta_bytes;
  t->d_values = mem.d_values;
  t->h_values = mem.h_values;
  t->view = nv;
  t->pure_hbm = nv.hbm_slots == nv.capacity;
  t->bounds_stale = true; /* the new arenas have none yet */
  free_arenas(t, old);
  return HKV_SUCCESS;
}

/* reserve, merlin_hashtable.cuh:3503-3541 */
int reserve_impl(hkv_table* t, uint64_t new_capacity, hipStream_t s) {
  if (t->reach_max_capacity || new_capacity > t->opts.max_capacity) {
    t->reach_max_capacity = t->view.capacity * 2 > t->opts.max_capacity;
    return HKV_SUCCESS;
  }
  {
    LockGuard g(t, StreamGroupLock::kInserter, s);
    HKV_HIP(g.acquire());
    /* with exclusive access, wait for everything that still uses the arenas */
    HKV_HIP(hipDeviceSynchronize());
    while (t->view.capacity < new_capacity && t->view.capacity * 2 <= t->opts.max_capacity)
      HKV_TRY(double_table(t, s));
    t->reach_max_capacity = t->view.capacity * 2 > t->opts.max_capacity;
  }
  return HKV_SUCCESS;
}

/* fast_load_factor, merlin_hashtable.cuh:3796-3830: the first min(buckets,
 * 1024) buckets stand for the table; the incoming batch counts as all new */
int fast_load_factor(hkv_table* t, uint64_t delta, hipStream_t s, float* out) {
  const uint32_t n = (uint32_t)std::min<uint64_t>(t->view.buckets_num, 1024);
  /* A word of its own, not one of the leased counters: callers that hold a lease come through
   * here (the count-returning insert_and_evict), and with all leases out they would wait for
   * each other.  The kernel stores its whole result in one write, so callers that overlap read
   * one or the other's sample of the same buckets, which serves the estimate as well. */
  unsigned long long* d = t->d_load_sample;
  {
    LockGuard g(t, StreamGroupLock::kReader, s);
    HKV_HIP(g.acquire());
    hipLaunchKernelGGL(load_sample_kernel, dim3(1), dim3(256), 0, s, t->view, n, d);
    HKV_HIP(hipGetLastError());
  }
  unsigned long long sum = 0;
  HKV_HIP(hipMemcpyAsync(&sum, d, sizeof sum, hipMemcpyDeviceToHost, s));
  HKV_HIP(hipStreamSynchronize(s));
  *out = (float)((delta * 1.0) / (t->view.capacity * 1.0) + (sum * 1.0) / (kBucketSize * n * 1.0));
  return HKV_SUCCESS;
}

/* the growth loop at the head of every inserting call
 * (merlin_hashtable.cuh:1151-1154, 1369-1372, 1604-1607, 1712-1715, 1898-1901) */
int grow_for(hkv_table* t, uint64_t n, hipStream_t s) {
  while (!t->reach_max_capacity) {
    float lf = 0.f;
    HKV_TRY(fast_load_factor(t, n, s, &lf));
    if (!(lf > t->opts.max_load_factor)) break;
    HKV_TRY(reserve_impl(t, t->view.capacity * 2, s));
  }
  return HKV_SUCCESS;
}

/* Slots left LOCKED between calls make the upserts scan key words beside the scores and keep
 * them off the two-phase path.  After an unlock_keys the device count is read once (the caller
 * holds the inserter role on `s`, so the unlock has been ordered before this point); at zero
 * the table is back to the plain kernels. */
int settle_locked_count(hkv_table* t, hipStream_t s) {
  if (!t->keys_may_be_locked || !t->locked_recount) return HKV_SUCCESS;
  static_assert(sizeof(long long) == sizeof(unsigned long long), "");
  std::vector<long long> words(kLockedShards * kLockedStride);
  HKV_HIP(hipMemcpyAsync(words.data(), t->d_locked, words.size() * sizeof(long long), hipMemcpyDeviceToHost, s));
  HKV_HIP(hipStreamSynchronize(s));
  long long left = 0; /* a shard may be below zero: keys are unlocked by other workgroups than locked them */
  for (unsigned k = 0; k < kLockedShards; k++) left += words[k * kLockedStride];
  t->locked_recount = false;
  if (left <= 0) t->keys_may_be_locked = false;
  return HKV_SUCCESS;
}

bool capturing(hipStream_t s) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(s, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st == hipStreamCaptureStatusActive;
}

/* A call that writes scores is about to run without looking after the score bounds (the plain
 * upsert kernels, the two-phase path, lock_keys / find_and_update, assign on a table whose
 * bounds are stale anyway).  The caller holds its role of the group lock, so this is ordered
 * with the upsert that next rebuilds the bounds.
 * - A call that is being recorded into a HIP graph runs again with every replay, at times the
 *   library knows nothing of, with the scores, epoch and clock base of the day it was recorded:
 *   from then on the table does without the bounds.
 * - LRU and EpochLRU scores come from the clock and only grow, whichever kernel writes them
 *   (`own_rule`: the call follows the table's strategy, i.e. no ignore_evict_strategy): the
 *   bounds stay right.  Every other score may be below a bound: they are made again before
 *   their next use. */
void writes_scores_outside_bounds(hkv_table* t, hipStream_t s, bool own_rule) {
  if (!t->score_bounds) return;
  const int st = t->opts.evict_strategy;
  if (capturing(s)) {
    /* (a replay of an LRU call on the hardware clock writes the time of the replay, which is as
     * good as any: such a table keeps its bounds; an epoch or a deterministic clock is recorded
     * with its value of today) */
    if (!(own_rule && st == HKV_LRU && t->clock.mode == 0)) t->score_bounds = false;
    return;
  }
  if (own_rule && (st == HKV_LRU || st == HKV_EPOCH_LRU)) return;
  t->bounds_stale = true;
}

uint64_t host_realtime_ns() {
  struct timespec ts;
  clock_gettime(CLOCK_REALTIME, &ts);
  return (uint64_t)ts.tv_sec * UINT64_C(1000000000) + (uint64_t)ts.tv_nsec;
}

/* Whether this upsert searches victims through the score bounds, and with which limits (the
 * fields of `a`); launches what has to run first (the batch's lowest score, the rebuild).  The
 * caller holds the inserter role on `s`. */
template <int OP>
bool prepare_bounds(hkv_table* t, UpsertArgs& a, int vec, hipStream_t s) {
  const int st = t->opts.evict_strategy;
  if (!t->score_bounds || a.strategy != st || !(vec == 16 || OP == kOpFindOrInsertPtr)) return false;
  /* The bounded search pays once buckets are full; a table that cannot be nine tenths full yet (it
   * has not been offered that many keys since it was created or cleared) takes the plain kernel. */
  if (t->keys_offered * 10 < t->view.capacity * 9) return false;
  if (capturing(s)) return false; /* writes_scores_outside_bounds() then switches the bounds off */
  const bool from_clock = st == HKV_LRU || st == HKV_EPOCH_LRU;
  if (st == HKV_EPOCH_LRU) {
    /* (epoch << 32) | (clock >> 20 & 0xFFFFFFFF) grows while the epoch does not go back and the low
     * half does not wrap (every 2^52 ns); a call that may see the wrap happen, or a clock that
     * cannot be read here, does without the bounds */
    const uint64_t now = t->clock.mode == 1 ? t->clock.base : host_realtime_ns();
    const uint64_t low = (now >> 20) & kLow32;
    const uint64_t margin = t->clock.mode == 1 ? a.n + 1 : (UINT64_C(1) << 14); /* 2^14 * 2^20 ns = 17 s */
    if (low + margin > kLow32 || (t->clock.mode == 0 && low < margin)) {
      t->bounds_stale = true;
      return false;
    }
    if (t->epoch < t->bounds_epoch || (t->epoch == t->bounds_epoch && (now >> 52) != t->bounds_era))
      t->bounds_stale = true;
    t->bounds_epoch = t->epoch;
    t->bounds_era = now >> 52;
  }
  BoundsRebuild r{};
  r.clock = t->clock;
  r.strategy = st;
  r.epoch = t->epoch;
  if (from_clock) {
    /* No bound may be above a score that this call writes.  Deterministic clock: the call's
     * scores start at its base.  Hardware clock: they are later than the start of the last
     * call of this kind, which that call left in a device word (this one leaves its own in
     * the other word). */
    a.bound_cap = t->clock.base;
    if (t->clock.mode == 0) {
      a.bound_cap_in = t->d_bound_caps + (t->bound_cap_turn & 1);
      a.bound_cap_out = t->d_bound_caps + ((t->bound_cap_turn + 1) & 1);
      t->bound_cap_turn++;
      r.clock_word = const_cast<unsigned long long*>(a.bound_cap_in);
    }
  } else {
    /* Scores from the caller: the limit is the lowest score this batch can leave behind, found
     * by a pass over its scores; keys that write a score below the limits of earlier calls
     * (d_bound_ceil) lower their line's bound themselves (hkv_upsert.hpp). */
    unsigned long long* floor_word = t->d_score_floor + (t->score_floor_turn & 1);
    unsigned long long* next_word = t->d_score_floor + ((t->score_floor_turn + 1) & 1);
    t->score_floor_turn++;
    const unsigned blocks = (unsigned)std::min<uint64_t>(64, (a.n + 8191) / 8192);
    hipLaunchKernelGGL(score_floor_kernel, dim3(blocks), dim3(1024), 0, s, a.scores, a.n, st, t->epoch,
                       floor_word, next_word);
    a.bound_cap_in = floor_word;
    a.bound_ceil = t->d_bound_ceil;
    r.floor_word = floor_word;
    r.ceil_word = t->d_bound_ceil;
  }
  /* bounds that were never set (a new or cleared table reaching this point) or that may be
   * above a score (scores from outside the clock) are made from the scores as they are */
  if (t->bounds_stale.exchange(false)) {
    const uint64_t threads = t->view.capacity / 16 * 8;
    hipLaunchKernelGGL(rebuild_bounds_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, s,
                       t->view, r);
  }
  return true;
}

/* `hybrid_rule`: the operation follows the lock-key kernels of hybrid mode when
 * the table is not pure HBM (insert_or_assign, find_or_insert); the pointer
 * overload always does. */
template <int OP>
int run_upsert(hkv_table* t, UpsertArgs a, int vec, bool hybrid_rule, hipStream_t s) {
  HKV_TRY(grow_for(t, a.n, s));
  a.epoch = t->epoch;
  a.clock = t->clock;
  a.value_kind = t->opts.value_kind;
  const bool refuse_equal = OP == kOpFindOrInsertPtr || (hybrid_rule && !t->pure_hbm);
  a.refuse_equal = refuse_equal;
  const bool own_rule = a.strategy == t->opts.evict_strategy;
  t->keys_offered += a.n;
  {
    LockGuard g(t, StreamGroupLock::kInserter, s);
    HKV_HIP(g.acquire());
    HKV_TRY(settle_locked_count(t, s));
    if (OP == kOpFindOrInsertPtr && a.locked_key_ptrs) t->keys_may_be_locked = true;
    /* a table that has been offered fewer keys than nine tenths of its slots evicts next to nothing */
    const bool pair = OP == kOpInsertAndEvict && t->keys_offered * 10 >= t->view.capacity * 9;
    /* Hybrid mode: the reference settles the keys of a batch with one kernel that leaves every
     * slot it took LOCKED and moves the rows with a second one that unlocks them
     * (upsert.cuh:1350-1595, find_or_insert.cuh:1417-1676), so no key of a batch ever takes the
     * slot of another key of the same batch: the later key sees that slot as LOCKED, which the
     * victim scan of these kernels passes over.  Here the rows move under the same lock; the
     * slots stay LOCKED until the kernel is done and a second launch opens them.  (A call that
     * is being recorded into a graph cannot ask for the list of slots: it releases each slot as
     * soon as its key is in, which is the same as handing the keys over one call at a time.) */
    const bool hold = hybrid_rule && !t->pure_hbm && !capturing(s) &&
                      (OP == kOpInsertOrAssign || OP == kOpFindOrInsert);
    uint64_t** held = nullptr;
    if (hold) {
      /* n slot addresses, then n scores */
      HKV_HIP(hipMallocAsync((void**)&held, a.n * 16, s));
      const hipError_t e = hipMemsetAsync(held, 0, a.n * 8, s);
      if (e != hipSuccess) {
        (void)hipFreeAsync(held, s);
        HKV_HIP(e);
      }
      a.locked_key_ptrs = held;
      a.held_scores = reinterpret_cast<uint64_t*>(held) + a.n;
      a.locked_count = nullptr; /* nothing stays LOCKED beyond this call */
    }
    if (t->keys_may_be_locked) {
      /* slots that lock_keys (or the pointer overload with locked_key_ptrs) left LOCKED must
       * be hidden from the victim scan, which then reads the key words beside the scores; with
       * no such slot the plain scan finds the same victims (a slot locked by another key of
       * the batch is retried instead of skipped) */
      writes_scores_outside_bounds(t, s, own_rule);
      launch_upsert_for<OP, true>(pair, vec, t->view, a, s);
    } else if (prepare_bounds<OP>(t, a, vec, s)) {
      launch_upsert_for<OP, false, true>(pair, vec, t->view, a, s);
    } else {
      writes_scores_outside_bounds(t, s, own_rule);
      launch_upsert_for<OP, false>(pair, vec, t->view, a, s);
    }
    hipError_t e = hipGetLastError();
    if (hold) {
      if (e == hipSuccess) {
        hipLaunchKernelGGL(open_held_kernel, dim3((unsigned)((a.n + 255) / 256)), dim3(256), 0, s, t->view, a.n,
                           (uint64_t* const*)held, a.held_scores, a.keys);
        e = hipGetLastError();
      }
      (void)hipFreeAsync(held, s);
    }
    HKV_HIP(e);
  }
  if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
  return HKV_SUCCESS;
}

/* ---- io_by_cpu: host threads move the value rows of the writers -----------------
 * merlin_hashtable.cuh:1275-1292 (insert_or_assign), 1820-1841 (find_or_insert),
 * 2175-2192 (assign), 2414-2431 (assign_values); write_by_cpu upsert.cuh:1711-1747,
 * read_or_write_by_cpu find_or_insert.cuh:1814-1855.  All rows of such a table are in
 * pinned host memory (max_hbm_for_vectors must be 0).  A kernel settles keys, scores and
 * digests and reports the row address of every accepted key; addresses and the caller's
 * rows are copied to the host, the stream is synchronised and up to 16 host threads copy
 * the rows; the role of the group lock is held until they are done.  The upserts follow
 * the plain kernels' rule (refuse when score < min), as the reference's do with this
 * option. */
struct CpuIoStage {
  uint8_t** ptrs;   /* n row addresses (device view of the pinned rows) */
  uint8_t* founds;  /* n flags */
  uint8_t* rows;    /* n caller rows */
};

int cpu_io_stage(hkv_table* t, uint64_t n, CpuIoStage& st) {
  const uint64_t vb = t->view.value_bytes;
  const uint64_t off_founds = n * 8, off_rows = (off_founds + n + 255) & ~UINT64_C(255);
  const uint64_t need = off_rows + n * vb;
  if (need > t->io_stage_bytes) {
    if (t->io_stage) (void)hipHostFree(t->io_stage);
    t->io_stage = nullptr;
    t->io_stage_bytes = 0;
    HKV_HIP(hipHostMalloc(&t->io_stage, need, hipHostMallocDefault));
    t->io_stage_bytes = need;
  }
  uint8_t* base = (uint8_t*)t->io_stage;
  st.ptrs = (uint8_t**)base;
  st.founds = base + off_founds;
  st.rows = base + off_rows;
  return HKV_SUCCESS;
}

/* an address the kernels reported -> the host's address of the same row */
inline uint8_t* cpu_io_host_row(const hkv_table* t, const uint8_t* p) {
  return (uint8_t*)t->h_values + (p - t->view.host_values);
}

/* direction per key: 0 skip, 1 caller row -> table, 2 table -> caller row */
template <class Dir>
void cpu_io_copy(const hkv_table* t, uint64_t n, const CpuIoStage& st, Dir dir) {
  const uint64_t vb = t->view.value_bytes;
  const unsigned workers = (unsigned)std::min<uint64_t>(16, (n + 4095) / 4096);
  auto work = [&](uint64_t lo, uint64_t hi) {
    for (uint64_t i = lo; i < hi; i++) {
      if (!st.ptrs[i]) continue;
      uint8_t* row = cpu_io_host_row(t, st.ptrs[i]);
      const int d = dir(i);
      if (d == 1)
        memcpy(row, st.rows + i * vb, vb);
      else if (d == 2)
        memcpy(st.rows + i * vb, row, vb);
    }
  };
  if (workers <= 1) {
    work(0, n);
    return;
  }
  std::vector<std::thread> th;
  const uint64_t per = (n + workers - 1) / workers;
  for (unsigned w = 0; w < workers; w++) {
    const uint64_t lo = std::min<uint64_t>(n, w * per), hi = std::min<uint64_t>(n, lo + per);
    if (lo < hi) th.emplace_back(work, lo, hi);
  }
  for (auto& x : th) x.join();
}

/* A key that took a slot may lose it to a later key of the same batch (evicted again);
 * its address is dropped, so the row is written by the key that owns the slot at the end.
 * Keys that only read their row (`readers`: the hits of find_or_insert) keep theirs. */
__global__ void cpu_io_owner_kernel(View v, const uint64_t* keys, uint8_t** ptrs,
                                    const uint8_t* readers, uint64_t n) {
  const uint64_t i = blockIdx.x * (uint64_t)blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint8_t* p = ptrs[i];
  if (!p || (readers && readers[i])) return;
  const uint64_t slot = v.hbm_slots + (uint64_t)(p - v.host_values) / v.value_bytes;
  if (ld_u64(v.keys + slot) != keys[i]) ptrs[i] = nullptr;
}

/* insert_or_assign (reads == false) and find_or_insert (reads == true) */
int cpu_io_upsert(hkv_table* t, UpsertArgs a, void* values, bool reads, hipStream_t s) {
  HKV_TRY(grow_for(t, a.n, s));
  const uint64_t n = a.n, vb = t->view.value_bytes;
  std::lock_guard<std::mutex> host_lock(t->io_mutex);
  CpuIoStage st{};
  HKV_TRY(cpu_io_stage(t, n, st));
  void* d_tmp = nullptr;
  HKV_HIP(hipMallocAsync(&d_tmp, n * 9, s));
  a.out_ptrs = (void**)d_tmp;
  a.founds = (uint8_t*)d_tmp + n * 8;
  a.epoch = t->epoch;
  a.clock = t->clock;
  a.value_kind = t->opts.value_kind;
  a.refuse_equal = 0;
  hipError_t e = hipSuccess;
  {
    LockGuard g(t, StreamGroupLock::kInserter, s);
    e = g.acquire();
    if (e == hipSuccess) e = hipMemsetAsync(d_tmp, 0, n * 9, s); /* reserved / refused keys: no address */
    if (e == hipSuccess) {
      writes_scores_outside_bounds(t, s, a.strategy == t->opts.evict_strategy);
      launch_upsert<kOpFindOrInsertPtr, true>(16, t->view, a, s);
      hipLaunchKernelGGL(cpu_io_owner_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s,
                         t->view, a.keys, (uint8_t**)d_tmp,
                         reads ? (const uint8_t*)d_tmp + n * 8 : nullptr, n);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(st.ptrs, d_tmp, n * 8, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipMemcpyAsync(st.founds, (uint8_t*)d_tmp + n * 8, n, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipMemcpyAsync(st.rows, values, n * vb, hipMemcpyDefault, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    if (e == hipSuccess) {
      if (reads) {
        /* every read before any write: a row that is read by one key and taken over by
         * another key of the batch still holds what it held before the call */
        cpu_io_copy(t, n, st, [&](uint64_t i) { return st.founds[i] ? 2 : 0; });
        cpu_io_copy(t, n, st, [&](uint64_t i) { return st.founds[i] ? 0 : 1; });
        e = hipMemcpyAsync(values, st.rows, n * vb, hipMemcpyDefault, s);
        if (e == hipSuccess) e = hipStreamSynchronize(s);
      } else {
        cpu_io_copy(t, n, st, [](uint64_t) { return 1; });
      }
    }
  }
  (void)hipFreeAsync(d_tmp, s);
  HKV_HIP(e);
  if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
  return HKV_SUCCESS;
}


/* The calls that refuse a dual-bucket table with a MERLIN_CHECK
 * (merlin_hashtable.cuh:1362, 1597, 1705, 1891, 2233, 2304, 2860, 2905, 3505) report
 * HKV_ERROR_CHECK.  The calls the reference leaves unguarded although they probe one bucket
 * only (assign, find*, the missed-keys find, lock_keys, unlock_keys, find_and_update) report
 * HKV_ERROR_UNSUPPORTED instead of answering wrongly. */
int refuse_dual(const hkv_table* t, const char* what, bool guarded) {
  if (!t->dual) return HKV_SUCCESS;
  return fail(guarded ? HKV_ERROR_CHECK : HKV_ERROR_UNSUPPORTED,
              "[MEMORY_MODE] %s is not supported in dual-bucket mode.", what);
}

/* unique_key == false: the batch is reduced to one occurrence per key first; `keys` then
 * points at the reduced copy, which lives until the guard goes out of scope (stream-ordered). */
struct DedupGuard {
  DedupPlan d;
  bool on = false;
  ~DedupGuard() {
    if (on) dedup_free(d);
  }
};
int maybe_dedup(const hkv_table* t, int unique_key, uint64_t n, const uint64_t*& keys,
                hipStream_t s, DedupGuard& g) {
  if (unique_key || n < 2) return HKV_SUCCESS;
  if (n >= (UINT64_C(1) << 31))
    return fail(HKV_ERROR_UNSUPPORTED, "unique_key = false needs a batch below 2^31 keys");
  const hipError_t e = dedup_make(t->view, n, keys, s, g.d);
  if (e != hipSuccess) return fail(HKV_ERROR_HIP, "duplicate-key pass: %s", hipGetErrorString(e));
  g.on = true;
  keys = g.d.keys;
  return HKV_SUCCESS;
}

/* Where a key lands depends on the bucket sizes the moment it is handled, and the keys in
 * flight at once decide on counts that miss each other's claims.  With many buckets that is
 * noise; on a small table (the reference tests 1024 buckets with batches of 2^17 keys) it
 * unbalances the two-choice placement enough to drop keys while free slots remain (size after
 * the first such batch 129 085 against 130 726 for keys handled one by one).  So a batch goes in
 * as launches of at most 16 keys per bucket: one launch for any table of realistic size. */
void launch_dual_upsert(int vec, const View& v, const UpsertArgs& whole, hipStream_t s) {
  const uint64_t chunk = std::max<uint64_t>(v.buckets_num * 16, 4096);
  for (uint64_t off = 0; off < whole.n; off += chunk) {
    UpsertArgs a = whole;
    a.n = std::min<uint64_t>(chunk, whole.n - off);
    a.keys += off;
    a.values_in += off * v.value_bytes;
    if (a.scores) a.scores += off;
    if (a.clock.mode == 1) a.clock.base += off << 20; /* the deterministic clock: base + (index << 20) */
    const dim3 grid((unsigned)((a.n + kTilesPerWave - 1) / kTilesPerWave)), block(kWave);
    if (vec == 16)
      hipLaunchKernelGGL((dual_upsert_kernel<16>), grid, block, 0, s, v, a);
    else if (vec == 4)
      hipLaunchKernelGGL((dual_upsert_kernel<4>), grid, block, 0, s, v, a);
    else
      hipLaunchKernelGGL((dual_upsert_kernel<1>), grid, block, 0, s, v, a);
  }
}

void launch_dual_lookup(int vec, const View& v, const FindArgs& a, hipStream_t s) {
  const dim3 grid(grid_for(a.n)), block(kWave);
  if (vec == 16)
    hipLaunchKernelGGL((lookup_kernel<kLookupValues, 16, true>), grid, block, 0, s, v, a);
  else if (vec == 4)
    hipLaunchKernelGGL((lookup_kernel<kLookupValues, 4, true>), grid, block, 0, s, v, a);
  else
    hipLaunchKernelGGL((lookup_kernel<kLookupValues, 1, true>), grid, block, 0, s, v, a);
}

template <int MODE>
void launch_lookup(int vec, const View& v, const FindArgs& a, hipStream_t s) {
  const dim3 grid(grid_for(a.n)), block(kWave);
  if (vec == 16)
    launch_main(lookup_kernel<MODE, 16>, grid, block, s, v, a);
  else if (vec == 4)
    launch_main(lookup_kernel<MODE, 4>, grid, block, s, v, a);
  else
    launch_main(lookup_kernel<MODE, 1>, grid, block, s, v, a);
}

/* the missed-keys find: 16 wavefronts per workgroup (see lookup_kernel) */
void launch_lookup_missed(int vec, const View& v, const FindArgs& a, hipStream_t s) {
  constexpr int kWaves = 16;
  const dim3 grid((unsigned)((a.n + kWave * kWaves - 1) / (kWave * kWaves))), block(kWave * kWaves);
  if (vec == 16)
    hipLaunchKernelGGL((lookup_kernel<kLookupValues, 16, false, kWaves>), grid, block, 0, s, v, a);
  else if (vec == 4)
    hipLaunchKernelGGL((lookup_kernel<kLookupValues, 4, false, kWaves>), grid, block, 0, s, v, a);
  else
    hipLaunchKernelGGL((lookup_kernel<kLookupValues, 1, false, kWaves>), grid, block, 0, s, v, a);
}

template <bool LOCKFREE>
void launch_assign(int vec, const View& v, const AssignArgs& a, hipStream_t s) {
  const dim3 grid(grid_for(a.n)), block(kWave);
  if (vec == 16) {
    switch (pick_upl(v.value_bytes, 16)) {
      case 1: hipLaunchKernelGGL((assign_kernel<16, 1, LOCKFREE>), grid, block, 0, s, v, a); break;
      case 2: hipLaunchKernelGGL((assign_kernel<16, 2, LOCKFREE>), grid, block, 0, s, v, a); break;
      case 4: hipLaunchKernelGGL((assign_kernel<16, 4, LOCKFREE>), grid, block, 0, s, v, a); break;
      default: hipLaunchKernelGGL((assign_kernel<16, 8, LOCKFREE>), grid, block, 0, s, v, a); break;
    }
  } else if (vec == 4) {
    hipLaunchKernelGGL((assign_kernel<4, 8, LOCKFREE>), grid, block, 0, s, v, a);
  } else {
    hipLaunchKernelGGL((assign_kernel<1, 8, LOCKFREE>), grid, block, 0, s, v, a);
  }
}

template <class Pred>
void launch_export(const hkv_table* t, uint64_t pattern, uint64_t threshold,
                   uint64_t n, uint64_t offset, uint64_t* d_counter,
                   uint64_t* keys, void* values, uint64_t* scores, hipStream_t s) {
  const unsigned blocks = export_grid(n, kExportThreads);
  hipLaunchKernelGGL((export_if_kernel<Pred>), dim3(blocks), dim3(kExportThreads), 0, s,
                     t->view, Pred(), pattern, threshold, offset, n,
                     (unsigned long long*)d_counter, keys, (uint8_t*)values, scores);
}

template <class Pred>
void launch_size_if(const hkv_table* t, uint64_t pattern, uint64_t threshold,
                    unsigned long long* d_out, hipStream_t s) {
  const unsigned blocks = scan_grid(t->view.capacity, 256);
  hipLaunchKernelGGL((size_if_kernel<Pred>), dim3(blocks), dim3(256), 0, s,
                     t->view, Pred(), pattern, threshold, d_out);
}

int create_impl(const hkv_options* o, const hkv_allocator* al, hkv_table** out) {
  if (!o || !out) return fail(HKV_ERROR_ARGUMENT, "null argument");
  /* HashTable::init, merlin_hashtable.cuh:1016-1048 */
  if (o->table_mode != 0 && o->table_mode != 1)
    return fail(HKV_ERROR_ARGUMENT, "bad table_mode %d", o->table_mode);
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
    if (o->dim * (uint64_t)o->value_size > 224 * sizeof(float))
      return fail(HKV_ERROR_CHECK,
                  "[MEMORY_MODE] dim * sizeof(V) must not exceed 896 bytes "
                  "(i.e. dim <= 224 for float).");
    if (o->max_bucket_size == 0 || o->init_capacity / o->max_bucket_size < 2)
      return fail(HKV_ERROR_CHECK,
                  "[MEMORY_MODE] capacity must provide at least 2 buckets "
                  "(capacity >= 2 * max_bucket_size).");
  }
  if (o->reserved_key_start_bit < 0 || o->reserved_key_start_bit > 62)
    return fail(HKV_ERROR_CHECK, "options.reserved_key_start_bit should >= 0 and <= 62.");
  if (!ispow2(o->max_bucket_size))
    return fail(HKV_ERROR_CHECK, "Bucket size should be the pow of 2");
  if (!ispow2(o->num_of_buckets_per_alloc))
    return fail(HKV_ERROR_CHECK, "Then `num_of_buckets_per_alloc` should be the pow of 2");
  if (o->init_capacity < o->num_of_buckets_per_alloc * o->max_bucket_size)
    return fail(HKV_ERROR_CHECK,
                "Then `num_of_buckets_per_alloc` must be equal or less than "
                "initial required buckets number");
  if (o->max_bucket_size != kBucketSize)
    return fail(HKV_ERROR_UNSUPPORTED, "only max_bucket_size == 128 is supported");
  if (o->io_by_cpu && o->max_hbm_for_vectors != 0)
    return fail(HKV_ERROR_CHECK,
                "[HierarchicalKV] `io_by_cpu` should not be true when "
                "`max_hbm_for_vectors` is not 0!");
  if (o->io_by_cpu && o->table_mode == 1)
    return fail(HKV_ERROR_UNSUPPORTED, "io_by_cpu is not supported in dual-bucket mode");
  if (o->evict_strategy < 0 || o->evict_strategy > 4)
    return fail(HKV_ERROR_ARGUMENT, "bad evict_strategy %d", o->evict_strategy);
  if (o->score_size != 8)
    return fail(HKV_ERROR_UNSUPPORTED, "only 64-bit scores are supported");
  if (o->dim == 0 || o->value_size == 0)
    return fail(HKV_ERROR_ARGUMENT, "dim and value_size must be positive");
  if (o->dim * (uint64_t)o->value_size > (1u << 20))
    return fail(HKV_ERROR_UNSUPPORTED, "value rows above 1 MiB are not supported");
  const uint32_t ksz[] = {0, 4, 8, 4, 8, 1, 2};
  if (o->value_kind < 0 || o->value_kind > 6 ||
      (o->value_kind != 0 && ksz[o->value_kind] != o->value_size))
    return fail(HKV_ERROR_ARGUMENT, "value_kind does not match value_size");

  hkv_table* t = new (std::nothrow) hkv_table();
  if (!t) return fail(HKV_ERROR_RUNTIME, "out of memory");
  t->opts = *o;
  t->own_alloc = al == nullptr;
  if (al) t->alloc = *al;
  t->d_meta = nullptr;
  t->d_values = nullptr;
  t->d_counters = nullptr;
  t->h_values = nullptr;
  t->keys_may_be_locked = false;
  t->locked_recount = false;
  t->dual = o->table_mode == 1;
  t->io_by_cpu = o->io_by_cpu != 0;
  t->io_stage = nullptr;
  t->io_stage_bytes = 0;
  {
    const char* b = getenv("HKV_SCORE_BOUNDS");
    /* dual-bucket tables have their own kernel, which scans both buckets; without the group
     * lock two upserts may run at once on two streams, and the limits of the bounds (the clock
     * reading or lowest score of "the call that is running") are kept per table, not per call */
    t->score_bounds = !(b && !strcmp(b, "0")) && !t->dual && o->api_lock != 0;
  }
  memset(&t->view, 0, sizeof t->view);
  t->epoch = kIgnoredEpoch;
  t->clock.base = 0;
  t->clock.offset = 0;
  t->clock.mode = 0;
  t->clock.ns_per_tick = 10;

  auto bail = [&](int rc) {
    std::string keep = g_err;
    hkv_table_destroy(t);
    g_err = keep;
    return rc;
  };

  if (o->device_id >= 0) {
    hipError_t e = hipSetDevice(o->device_id);
    if (e != hipSuccess) return bail(fail(HKV_ERROR_HIP, "hipSetDevice: %s", hipGetErrorString(e)));
    t->device = o->device_id;
  } else {
    hipError_t e = hipGetDevice(&t->device);
    if (e != hipSuccess) return bail(fail(HKV_ERROR_HIP, "hipGetDevice: %s", hipGetErrorString(e)));
    t->opts.device_id = t->device;
  }
  int khz = 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, t->device) == hipSuccess &&
      khz > 0)
    t->clock.ns_per_tick = (uint32_t)std::max(1, 1000000 / khz);

  View& v = t->view;
  /* create_table, core_kernels.cuh:343-357 */
  const uint64_t max_size = std::max(o->init_capacity, o->max_capacity);
  if (o->init_capacity * 2 > max_size) {
    v.buckets_num = 1 + (max_size - 1) / kBucketSize;
  } else {
    v.buckets_num = 1;
    while (v.buckets_num * kBucketSize < o->init_capacity) v.buckets_num *= 2;
  }
  if (v.buckets_num >= (UINT64_C(1) << 31))
    return bail(fail(HKV_ERROR_UNSUPPORTED, "more than 2^31 buckets"));
  v.capacity = v.buckets_num * kBucketSize;
  v.pow2_buckets = ispow2(v.buckets_num);
  v.dim = (uint32_t)o->dim;
  v.value_bytes = (uint32_t)(o->dim * o->value_size);
  /* init_reserved_keys, types.cuh:80-109 */
  const int b = o->reserved_key_start_bit;
  if (b == 0) {
    v.empty_key = UINT64_C(0xFFFFFFFFFFFFFFFF);
    v.reclaim_key = UINT64_C(0xFFFFFFFFFFFFFFFE);
    v.locked_key = UINT64_C(0xFFFFFFFFFFFFFFFD);
    v.reserved_mask1 = v.reserved_mask2 = UINT64_C(0xFFFFFFFFFFFFFFFC);
  } else {
    v.reserved_mask1 = ~(UINT64_C(3) << b);
    v.reserved_mask2 = v.reserved_mask1 & ~UINT64_C(1);
    v.empty_key = v.reserved_mask2 | (UINT64_C(3) << b);
    v.reclaim_key = ~(UINT64_C(1) << b) & ~UINT64_C(1);
    v.locked_key = v.empty_key & ~(UINT64_C(2) << b);
  }
  v.empty_digest = (uint8_t)(fmix64(v.empty_key) >> 32);
  v.reclaim_digest = (uint8_t)(fmix64(v.reclaim_key) >> 32);
  if (t->dual) {
    /* dual_bucket_empty_digest, dual_bucket_utils.cuh:86-90; core_kernels.cuh:67-71 */
    v.empty_digest = (uint8_t)(fmix64(v.empty_key) >> 56);
    v.reclaim_digest = (uint8_t)(fmix64(v.reclaim_key) >> 56);
  }
  v.dual_bucket = t->dual ? 1 : 0;

  TableMem mem{};
  {
    int rc = alloc_arenas(t, v.buckets_num, v, mem);
    if (rc) {
      free_arenas(t, mem);
      return bail(rc);
    }
  }
  t->d_meta = mem.d_meta;
  t->meta_bytes = mem.meta_bytes;
  t->d_values = mem.d_values;
  t->h_values = mem.h_values;
  t->pure_hbm = v.hbm_slots == v.capacity;
  void* cnt = nullptr;
  {
    int rc = table_alloc(t, 0, &cnt, (kCounterWords + kExtraWords) * sizeof(unsigned long long));
    if (rc) return bail(rc);
  }
  t->d_counters = (unsigned long long*)cnt;
  for (unsigned w = 0; w < kCounterWords; w++) t->counter_free.push_back(w);
  t->d_bound_caps = t->d_counters + kCounterWords;
  t->d_score_floor = t->d_counters + kCounterWords + 2;
  t->d_bound_ceil = t->d_counters + kCounterWords + 4;
  t->d_load_sample = t->d_counters + kCounterWords + 5;
  t->d_locked = t->d_counters + kCounterWords + 8;
  {
    int rc = sync_clock(t);
    if (rc) return bail(rc);
    /* score_floor_kernel takes the minimum into a word that holds the highest score */
    if (hipMemset(t->d_score_floor, 0xFF, 2 * sizeof(unsigned long long)) != hipSuccess)
      return bail(fail(HKV_ERROR_HIP, "hipMemset of the score floor words failed"));
  }
  t->reach_max_capacity = t->dual || o->init_capacity * 2 > o->max_capacity; /* merlin_hashtable.cuh:1064-1069 */
  *out = t;
  return HKV_SUCCESS;
}

}  // namespace

extern "C" {

void hkv_options_default(hkv_options* o) {
  memset(o, 0, sizeof *o);
  o->max_bucket_size = 128;
  o->dim = 64;
  o->max_load_factor = 0.5f;
  o->block_size = 128;
  o->io_block_size = 1024;
  o->device_id = -1;
  o->num_of_buckets_per_alloc = 1;
  o->api_lock = 1;
  o->evict_strategy = HKV_LRU;
  o->value_kind = HKV_VALUE_F32;
  o->value_size = 4;
  o->score_size = 8;
}

const char* hkv_last_error(void) { return g_err.c_str(); }
const char* hkv_version(void) { return "hkv-amd 0.1 (gfx950)"; }

int hkv_table_create(const hkv_options* opts, hkv_table** out) {
  return create_impl(opts, nullptr, out);
}

int hkv_table_create_with_allocator(const hkv_options* opts,
                                    const hkv_allocator* allocator,
                                    hkv_table** out) {
  if (!allocator || !allocator->alloc || !allocator->free)
    return fail(HKV_ERROR_ARGUMENT, "allocator callbacks must not be null");
  return create_impl(opts, allocator, out);
}

int hkv_table_destroy(hkv_table* t) {
  if (!t) return HKV_SUCCESS;
  (void)hipSetDevice(t->device);
  (void)hipDeviceSynchronize();
  table_free(t, 0, t->d_meta);
  table_free(t, 0, t->d_counters);
  table_free(t, 0, t->d_values);
  table_free(t, 1, t->h_values);
  if (t->io_stage) (void)hipHostFree(t->io_stage);
  delete t;
  return HKV_SUCCESS;
}

int hkv_insert_or_assign(hkv_table* t, uint64_t n, const uint64_t* keys,
                         const void* values, const uint64_t* scores,
                         hkv_stream_t stream, int unique_key, int ignore) {
  if (n == 0) return HKV_SUCCESS;
  const int strategy = ignore ? HKV_CUSTOMIZED : t->opts.evict_strategy;
  if (!ignore) HKV_TRY(check_scores_arg(t, strategy, scores));
  DedupGuard dg;
  if (!t->dual) HKV_TRY(maybe_dedup(t, unique_key, n, keys, (hipStream_t)stream, dg));
  UpsertArgs a{};
  a.keys = keys;
  a.values_in = (const uint8_t*)values;
  a.scores = scores;
  a.n = n;
  a.strategy = strategy;
  const int vec = pick_vec(t->view.value_bytes, {values});
  if (t->dual) {
    /* merlin_hashtable.cuh:1166-1190 */
    if (!unique_key)
      return fail(HKV_ERROR_CHECK,
                  "[MEMORY_MODE] insert_or_assign requires unique_key=true in dual-bucket mode.");
    hipStream_t s = (hipStream_t)stream;
    a.epoch = t->epoch;
    a.clock = t->clock;
    a.value_kind = t->opts.value_kind;
    {
      LockGuard g(t, StreamGroupLock::kInserter, s);
      HKV_HIP(g.acquire());
      launch_dual_upsert(vec, t->view, a, s);
      HKV_HIP(hipGetLastError());
    }
    if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
    return HKV_SUCCESS;
  }
  if (t->io_by_cpu) return cpu_io_upsert(t, a, const_cast<void*>(values), false, (hipStream_t)stream);
  /* with unique_key == false the reference leaves its lock-key kernels for the plain one
   * (merlin_hashtable.cuh:1235-1258), whose rule is "refuse when score < min" */
  return run_upsert<kOpInsertOrAssign>(t, a, vec, unique_key != 0, (hipStream_t)stream);
}

int hkv_insert_or_assign_noalloc(hkv_table* t, uint64_t n, const uint64_t* keys,
                                 const void* values, const uint64_t* scores,
                                 hkv_stream_t stream, int ignore) {
  if (n == 0) return HKV_SUCCESS;
  if (n > kNoAllocMaxKeys)
    return fail(HKV_ERROR_ARGUMENT, "hkv_insert_or_assign_noalloc: %llu keys, the limit is %llu per call",
                (unsigned long long)n, (unsigned long long)kNoAllocMaxKeys);
  if (t->view.buckets_num > kNoAllocMaxBuckets)
    return fail(HKV_ERROR_UNSUPPORTED,
                "hkv_insert_or_assign_noalloc: the table has %llu buckets, the limit is %llu",
                (unsigned long long)t->view.buckets_num, (unsigned long long)kNoAllocMaxBuckets);
  if (t->dual || t->io_by_cpu || !t->opts.api_lock)
    return fail(HKV_ERROR_UNSUPPORTED,
                "hkv_insert_or_assign_noalloc needs a single-bucket table with api_lock and without io_by_cpu");
  if (!t->reach_max_capacity)
    return fail(HKV_ERROR_UNSUPPORTED,
                "hkv_insert_or_assign_noalloc: the table can still grow, and growing allocates; "
                "reserve() it to max_capacity first");
  const int strategy = ignore ? HKV_CUSTOMIZED : t->opts.evict_strategy;
  if (!ignore) HKV_TRY(check_scores_arg(t, strategy, scores));
  hipStream_t s = (hipStream_t)stream;
  DeviceGuard dev(t->device);
  if (!dev.ok) return fail(HKV_ERROR_HIP, "cannot make device %d current", t->device);
  uint32_t* scratch = nullptr;
  HKV_TRY(noalloc_scratch(t->device, &scratch));
  UpsertArgs a{};
  a.keys = keys;
  a.values_in = (const uint8_t*)values;
  a.scores = scores;
  a.n = n;
  a.strategy = strategy;
  a.epoch = t->epoch;
  a.clock = t->clock;
  a.value_kind = t->opts.value_kind;
  a.refuse_equal = !t->pure_hbm; /* the lock-key rule of hybrid mode, as hkv_insert_or_assign */
  const int vec = pick_vec(t->view.value_bytes, {values});
  {
    LockGuard g(t, StreamGroupLock::kInserter, s);
    HKV_HIP(g.acquire());
    writes_scores_outside_bounds(t, s, a.strategy == t->opts.evict_strategy);
    /* slots left LOCKED by lock_keys are invisible to the second phase; whether any are left
     * after unlock_keys is settled by the next ordinary upsert (it reads a device counter) */
    if (t->keys_may_be_locked)
      return fail(HKV_ERROR_UNSUPPORTED,
                  "hkv_insert_or_assign_noalloc: keys may be locked (lock_keys / find_or_insert with "
                  "locked_key_ptrs)");
    ChainArgs c{};
    c.head = scratch;
    c.next = scratch + kNoAllocMaxBuckets;
    c.locked_rule = a.refuse_equal;
    /* the array keeps what the last call on this device left in it (all zero after a call
     * that ran to its end, but a call may have failed half way): the heads start at zero */
    const uint64_t head_words = (t->view.buckets_num + 3) & ~UINT64_C(3);
    hipLaunchKernelGGL(zero_words_kernel, dim3((unsigned)((head_words / 4 + 255) / 256)), dim3(256), 0, s,
                       c.head, head_words);
    dispatch_vec_upl<LaunchHits>(vec, t->view.value_bytes, t->view, a, c, s);
    dispatch_vec_upl<LaunchMisses>(vec, t->view.value_bytes, t->view, a, c, s);
    HKV_HIP(hipGetLastError());
  }
  if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
  return HKV_SUCCESS;
}

int hkv_insert_and_evict(hkv_table* t, uint64_t n, const uint64_t* keys,
                         const void* values, const uint64_t* scores,
                         uint64_t* evicted_keys, void* evicted_values,
                         uint64_t* evicted_scores, uint64_t* d_evicted_counter,
                         hkv_stream_t stream, int unique_key, int ignore) {
  HKV_TRY(refuse_dual(t, "insert_and_evict()", true));
  if (n == 0) return HKV_SUCCESS;
  /* merlin_hashtable.cuh:1384-1386 */
  if (!t->pure_hbm)
    return fail(HKV_ERROR_RUNTIME, "Only support pure HBM mode for insert_and_evict.");
  const int strategy = ignore ? HKV_CUSTOMIZED : t->opts.evict_strategy;
  if (!ignore) HKV_TRY(check_scores_arg(t, strategy, scores));
  DedupGuard dg;
  HKV_TRY(maybe_dedup(t, unique_key, n, keys, (hipStream_t)stream, dg));
  UpsertArgs a{};
  a.keys = keys;
  a.values_in = (const uint8_t*)values;
  a.scores = scores;
  a.evicted_keys = evicted_keys;
  a.evicted_values = (uint8_t*)evicted_values;
  a.evicted_scores = evicted_scores;
  a.evicted_counter = (unsigned long long*)d_evicted_counter;
  a.n = n;
  a.strategy = strategy;
  const int vec = pick_vec(t->view.value_bytes, {values, evicted_values});
  return run_upsert<kOpInsertAndEvict>(t, a, vec, false, (hipStream_t)stream);
}

int hkv_insert_and_evict_count(hkv_table* t, uint64_t n, const uint64_t* keys,
                               const void* values, const uint64_t* scores,
                               uint64_t* evicted_keys, void* evicted_values,
                               uint64_t* evicted_scores, hkv_stream_t stream,
                               int unique_key, int ignore, uint64_t* n_evicted) {
  HKV_TRY(refuse_dual(t, "insert_and_evict()", true));
  *n_evicted = 0;
  if (n == 0) return HKV_SUCCESS;
  hipStream_t s = (hipStream_t)stream;
  CounterLease lease(t, s);
  unsigned long long* d = lease.word();
  hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(1), 0, s, d);
  HKV_TRY(hkv_insert_and_evict(t, n, keys, values, scores, evicted_keys,
                               evicted_values, evicted_scores, (uint64_t*)d,
                               stream, unique_key, ignore));
  return lease.read(n_evicted);
}

int hkv_accum_or_assign(hkv_table* t, uint64_t n, const uint64_t* keys,
                        const void* value_or_deltas, const uint8_t* flags,
                        const uint64_t* scores, hkv_stream_t stream, int ignore) {
  HKV_TRY(refuse_dual(t, "accum_or_assign()", true));
  if (n == 0) return HKV_SUCCESS;
  if (t->opts.value_kind == HKV_VALUE_BYTES)
    return fail(HKV_ERROR_ARGUMENT, "accum_or_assign needs an arithmetic value_kind");
  const int strategy = ignore ? HKV_CUSTOMIZED : t->opts.evict_strategy;
  if (!ignore) HKV_TRY(check_scores_arg(t, strategy, scores));
  UpsertArgs a{};
  a.keys = keys;
  a.values_in = (const uint8_t*)value_or_deltas;
  a.accum_flags = flags;
  a.scores = scores;
  a.n = n;
  a.strategy = strategy;
  const int vec = accum_unit(t->view.value_bytes, value_or_deltas, t->opts.value_kind);
  if (vec == 0)
    return fail(HKV_ERROR_ARGUMENT, "accum_or_assign: value_or_deltas is not aligned to its element type");
  return run_upsert<kOpAccumOrAssign>(t, a, vec, false, (hipStream_t)stream);
}

int hkv_find_or_insert(hkv_table* t, uint64_t n, const uint64_t* keys,
                       void* values, const uint64_t* scores, hkv_stream_t stream,
                       int unique_key, int ignore) {
  HKV_TRY(refuse_dual(t, "find_or_insert()", true));
  if (n == 0) return HKV_SUCCESS;
  const int strategy = ignore ? HKV_CUSTOMIZED : t->opts.evict_strategy;
  if (!ignore) HKV_TRY(check_scores_arg(t, strategy, scores));
  DedupGuard dg;
  HKV_TRY(maybe_dedup(t, unique_key, n, keys, (hipStream_t)stream, dg));
  UpsertArgs a{};
  a.keys = keys;
  a.values_io = (uint8_t*)values;
  a.scores = scores;
  a.n = n;
  a.strategy = strategy;
  const int vec = pick_vec(t->view.value_bytes, {values});
  if (t->io_by_cpu)
    HKV_TRY(cpu_io_upsert(t, a, values, true, (hipStream_t)stream));
  else /* merlin_hashtable.cuh:1779-1803: lock-key kernels only with unique keys */
    HKV_TRY(run_upsert<kOpFindOrInsert>(t, a, vec, unique_key != 0, (hipStream_t)stream));
  if (dg.on) {
    /* the other occurrences of a key get the row its representative ended up with (what it
     * read, or what it inserted; a refused key keeps its own row, like its representative) */
    hipLaunchKernelGGL(dedup_fix_rows_kernel, dim3((unsigned)n), dim3(64), 0, (hipStream_t)stream,
                       (const uint32_t*)dg.d.rep, n, (uint8_t*)values, t->view.value_bytes);
    HKV_HIP(hipGetLastError());
  }
  return HKV_SUCCESS;
}

int hkv_find_or_insert_ptr_lock(hkv_table* t, uint64_t n, const uint64_t* keys, void** values,
                                uint8_t* founds, const uint64_t* scores,
                                uint64_t** locked_key_ptrs, hkv_stream_t stream, int ignore) {
  HKV_TRY(refuse_dual(t, "find_or_insert()", true));
  if (!locked_key_ptrs) return fail(HKV_ERROR_ARGUMENT, "locked_key_ptrs is null");
  if (n == 0) return HKV_SUCCESS;
  const int strategy = ignore ? HKV_CUSTOMIZED : t->opts.evict_strategy;
  if (!ignore) HKV_TRY(check_scores_arg(t, strategy, scores));
  UpsertArgs a{};
  a.keys = keys;
  a.out_ptrs = values;
  a.founds = founds;
  a.scores = scores;
  a.locked_key_ptrs = locked_key_ptrs;
  a.n = n;
  a.strategy = strategy;
  a.locked_count = t->d_locked; /* LOCKED key words stay behind until unlock_keys */
  return run_upsert<kOpFindOrInsertPtr>(t, a, 16, true, (hipStream_t)stream);
}

int hkv_find_or_insert_ptr(hkv_table* t, uint64_t n, const uint64_t* keys,
                           void** values, uint8_t* founds, const uint64_t* scores,
                           hkv_stream_t stream, int unique_key, int ignore) {
  HKV_TRY(refuse_dual(t, "find_or_insert()", true));
  if (n == 0) return HKV_SUCCESS;
  const int strategy = ignore ? HKV_CUSTOMIZED : t->opts.evict_strategy;
  if (!ignore) HKV_TRY(check_scores_arg(t, strategy, scores));
  DedupGuard dg;
  HKV_TRY(maybe_dedup(t, unique_key, n, keys, (hipStream_t)stream, dg));
  UpsertArgs a{};
  a.keys = keys;
  a.out_ptrs = values;
  a.founds = founds;
  a.scores = scores;
  a.n = n;
  a.strategy = strategy;
  HKV_TRY(run_upsert<kOpFindOrInsertPtr>(t, a, 16, true, (hipStream_t)stream));
  if (dg.on) {
    hipLaunchKernelGGL(dedup_fix_ptrs_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0,
                       (hipStream_t)stream, (const uint32_t*)dg.d.rep, n, values, founds);
    HKV_HIP(hipGetLastError());
  }
  return HKV_SUCCESS;
}

/* The group lock keeps every other writer off the table while an updater runs; with unique
 * keys the kernel then needs no slot locks.  Without the group lock (api_lock == false) other
 * streams may carry updaters the library knows nothing of, and a repeated key has two tiles
 * on one slot: both keep the slot locks. */
static int assign_common(hkv_table* t, uint64_t n, const uint64_t* keys,
                         const void* values, const uint64_t* scores,
                         int touch_scores, int unique_key, hipStream_t s) {
  const bool lockfree = t->opts.api_lock && unique_key;
  AssignArgs a{};
  a.keys = keys;
  a.values = (const uint8_t*)values;
  a.scores = scores;
  a.n = n;
  a.epoch = t->epoch;
  a.clock = t->clock;
  a.touch_scores = touch_scores;
  a.strategy = t->opts.evict_strategy;
  const int vec = pick_vec(t->view.value_bytes, {values});
  if (t->io_by_cpu && values) {
    /* scores by the kernel, row addresses by a lookup, rows by host threads */
    const uint64_t vb = t->view.value_bytes;
    std::lock_guard<std::mutex> host_lock(t->io_mutex);
    CpuIoStage st{};
    HKV_TRY(cpu_io_stage(t, n, st));
    void* d_tmp = nullptr;
    HKV_HIP(hipMallocAsync(&d_tmp, n * 9, s));
    hipError_t e = hipSuccess;
    {
      LockGuard g(t, StreamGroupLock::kUpdater, s);
      e = g.acquire();
      if (e == hipSuccess && touch_scores) {
        a.values = nullptr;
        writes_scores_outside_bounds(t, s, true);
        launch_assign<false>(16, t->view, a, s);
        e = hipGetLastError();
      }
      if (e == hipSuccess) e = hipMemsetAsync(d_tmp, 0, n * 9, s); /* reserved keys: no address */
      if (e == hipSuccess) {
        FindArgs f{};
        f.keys = keys;
        f.out_ptrs = (void**)d_tmp;
        f.founds = (uint8_t*)d_tmp + n * 8;
        f.n = n;
        launch_lookup<kLookupPtr>(16, t->view, f, s);
        e = hipGetLastError();
      }
      if (e == hipSuccess) e = hipMemcpyAsync(st.ptrs, d_tmp, n * 8, hipMemcpyDeviceToHost, s);
      if (e == hipSuccess) e = hipMemcpyAsync(st.rows, values, n * vb, hipMemcpyDefault, s);
      if (e == hipSuccess) e = hipStreamSynchronize(s);
      if (e == hipSuccess) cpu_io_copy(t, n, st, [](uint64_t) { return 1; });
    }
    (void)hipFreeAsync(d_tmp, s);
    HKV_HIP(e);
    if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
    return HKV_SUCCESS;
  }
  {
    LockGuard g(t, StreamGroupLock::kUpdater, s);
    HKV_HIP(g.acquire());
    /* Customized: the caller's score replaces the old one and may be below the line's bound;
     * EpochLFU: so may the old count under today's epoch, if the key carries a later one */
    if (t->score_bounds && touch_scores && scores &&
        (a.strategy == HKV_CUSTOMIZED || a.strategy == HKV_EPOCH_LFU)) {
      if (t->bounds_stale || capturing(s))
        writes_scores_outside_bounds(t, s, true);
      else
        a.bound_ceil = t->d_bound_ceil;
    }
    if (lockfree)
      launch_assign<true>(vec, t->view, a, s);
    else
      launch_assign<false>(vec, t->view, a, s);
    HKV_HIP(hipGetLastError());
  }
  if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
  return HKV_SUCCESS;
}

int hkv_assign(hkv_table* t, uint64_t n, const uint64_t* keys, const void* values,
               const uint64_t* scores, hkv_stream_t stream, int unique_key) {
  HKV_TRY(refuse_dual(t, "assign()", false));
  if (n == 0) return HKV_SUCCESS;
  HKV_TRY(check_scores_arg(t, t->opts.evict_strategy, scores));
  return assign_common(t, n, keys, values, scores, 1, unique_key, (hipStream_t)stream);
}

int hkv_assign_scores(hkv_table* t, uint64_t n, const uint64_t* keys,
                      const uint64_t* scores, hkv_stream_t stream, int unique_key) {
  HKV_TRY(refuse_dual(t, "assign_scores()", true));
  if (n == 0) return HKV_SUCCESS;
  HKV_TRY(check_scores_arg(t, t->opts.evict_strategy, scores));
  return assign_common(t, n, keys, nullptr, scores, 1, unique_key, (hipStream_t)stream);
}

int hkv_assign_values(hkv_table* t, uint64_t n, const uint64_t* keys,
                      const void* values, hkv_stream_t stream, int unique_key) {
  HKV_TRY(refuse_dual(t, "assign_values()", true));
  if (n == 0) return HKV_SUCCESS;
  return assign_common(t, n, keys, values, nullptr, 0, unique_key, (hipStream_t)stream);
}

int hkv_find(const hkv_table* t, uint64_t n, const uint64_t* keys, void* values,
             uint8_t* founds, uint64_t* scores, hkv_stream_t stream) {
  if (n == 0) return HKV_SUCCESS;
  hipStream_t s = (hipStream_t)stream;
  FindArgs a{};
  a.keys = keys;
  a.out_values = (uint8_t*)values;
  a.founds = founds;
  a.out_scores = scores;
  a.n = n;
  const int vec = pick_vec(t->view.value_bytes, {values});
  LockGuard g(t, StreamGroupLock::kReader, s);
  HKV_HIP(g.acquire());
  if (t->dual)
    launch_dual_lookup(vec, t->view, a, s);
  else
    launch_lookup<kLookupValues>(vec, t->view, a, s);
  HKV_HIP(hipGetLastError());
  return HKV_SUCCESS;
}

int hkv_find_missed(const hkv_table* t, uint64_t n, const uint64_t* keys,
                    void* values, uint64_t* missed_keys, int32_t* missed_indices,
                    int32_t* missed_size, uint64_t* scores, hkv_stream_t stream) {
  HKV_TRY(refuse_dual(t, "find() with the missed-keys outputs", false));
  if (n == 0) return HKV_SUCCESS;
  hipStream_t s = (hipStream_t)stream;
  FindArgs a{};
  a.keys = keys;
  a.out_values = (uint8_t*)values;
  a.out_scores = scores;
  a.missed_keys = missed_keys;
  a.missed_indices = missed_indices;
  a.missed_size = missed_size;
  a.n = n;
  const int vec = pick_vec(t->view.value_bytes, {values});
  hipLaunchKernelGGL(zero_i32_kernel, dim3(1), dim3(1), 0, s, missed_size);
  LockGuard g(t, StreamGroupLock::kReader, s);
  HKV_HIP(g.acquire());
  launch_lookup_missed(vec, t->view, a, s);
  HKV_HIP(hipGetLastError());
  return HKV_SUCCESS;
}

int hkv_find_ptr(const hkv_table* t, uint64_t n, const uint64_t* keys,
                 void** values, uint8_t* founds, uint64_t* scores,
                 hkv_stream_t stream, int unique_key) {
  HKV_TRY(refuse_dual(t, "find() by pointer", false));
  (void)unique_key;
  if (n == 0) return HKV_SUCCESS;
  hipStream_t s = (hipStream_t)stream;
  FindArgs a{};
  a.keys = keys;
  a.out_ptrs = values;
  a.founds = founds;
  a.out_scores = scores;
  a.n = n;
  LockGuard g(t, StreamGroupLock::kReader, s);
  HKV_HIP(g.acquire());
  launch_lookup<kLookupPtr>(16, t->view, a, s);
  HKV_HIP(hipGetLastError());
  return HKV_SUCCESS;
}

int hkv_contains(const hkv_table* t, uint64_t n, const uint64_t* keys,
                 uint8_t* founds, hkv_stream_t stream) {
  HKV_TRY(refuse_dual(t, "contains()", true));
  if (n == 0) return HKV_SUCCESS;
  hipStream_t s = (hipStream_t)stream;
  FindArgs a{};
  a.keys = keys;
  a.founds = founds;
  a.n = n;
  LockGuard g(t, StreamGroupLock::kReader, s);
  HKV_HIP(g.acquire());
  launch_lookup<kLookupContains>(16, t->view, a, s);
  HKV_HIP(hipGetLastError());
  return HKV_SUCCESS;
}

int hkv_lock_keys(hkv_table* t, uint64_t n, const uint64_t* keys, uint64_t** locked_key_ptrs,
                  uint8_t* success, const uint64_t* scores, hkv_stream_t stream) {
  HKV_TRY(refuse_dual(t, "lock_keys()", false));
  if (n == 0) return HKV_SUCCESS;
  HKV_TRY(check_scores_arg(t, t->opts.evict_strategy, scores));
  hipStream_t s = (hipStream_t)stream;
  TouchArgs a{};
  a.keys = keys;
  a.scores = const_cast<uint64_t*>(scores);
  a.key_ptrs = locked_key_ptrs;
  a.flags = success;
  a.locked_count = t->d_locked;
  a.n = n;
  a.epoch = t->epoch;
  a.clock = t->clock;
  a.strategy = t->opts.evict_strategy;
  {
    LockGuard g(t, StreamGroupLock::kInserter, s);
    HKV_HIP(g.acquire());
    t->keys_may_be_locked = true;
    writes_scores_outside_bounds(t, s, true);
    hipLaunchKernelGGL((touch_kernel<true>), dim3(grid_for(n)), dim3(kWave), 0, s, t->view, a);
    HKV_HIP(hipGetLastError());
  }
  if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
  return HKV_SUCCESS;
}

int hkv_unlock_keys(hkv_table* t, uint64_t n, uint64_t** locked_key_ptrs, const uint64_t* keys,
                    uint8_t* success, hkv_stream_t stream) {
  HKV_TRY(refuse_dual(t, "unlock_keys()", false));
  if (n == 0) return HKV_SUCCESS;
  hipStream_t s = (hipStream_t)stream;
  LockGuard g(t, StreamGroupLock::kInserter, s);
  HKV_HIP(g.acquire());
  hipLaunchKernelGGL(unlock_keys_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, t->view,
                     n, locked_key_ptrs, keys, success, t->d_locked);
  HKV_HIP(hipGetLastError());
  t->locked_recount = true;
  return HKV_SUCCESS;
}

int hkv_find_and_update(hkv_table* t, uint64_t n, const uint64_t* keys, void** values,
                        uint8_t* founds, uint64_t* scores, hkv_stream_t stream) {
  HKV_TRY(refuse_dual(t, "find_and_update()", false));
  if (n == 0) return HKV_SUCCESS;
  HKV_TRY(check_scores_arg(t, t->opts.evict_strategy, scores));
  hipStream_t s = (hipStream_t)stream;
  TouchArgs a{};
  a.keys = keys;
  a.scores = scores;
  a.value_ptrs = values;
  a.flags = founds;
  a.n = n;
  a.epoch = t->epoch;
  a.clock = t->clock;
  a.strategy = t->opts.evict_strategy;
  {
    /* it writes scores, so it runs with the updaters, not with the readers */
    LockGuard g(t, StreamGroupLock::kUpdater, s);
    HKV_HIP(g.acquire());
    hipLaunchKernelGGL((touch_kernel<false>), dim3(grid_for(n)), dim3(kWave), 0, s, t->view, a);
    HKV_HIP(hipGetLastError());
  }
  if (t->clock.mode == 1) t->clock.base += UINT64_C(1) << 40;
  return HKV_SUCCESS;
}

int hkv_erase(hkv_table* t, uint64_t n, const uint64_t* keys, hkv_stream_t stream) {
  HKV_TRY(refuse_dual(t, "erase()", true));
  if (n == 0) return HKV_SUCCESS;
  hipStream_t s = (hipStream_t)stream;
  LockGuard g(t, StreamGroupLock::kInserter, s);
  HKV_HIP(g.acquire());
  /* with the group lock on, the inserter role makes this call the only one on the table */
  if (t->opts.api_lock)
    hipLaunchKernelGGL(erase_kernel<true>, dim3(grid_for(n)), dim3(kWave), 0, s, t->view, keys, n);
  else
    hipLaunchKernelGGL(erase_kernel<false>, dim3(grid_for(n)), dim3(kWave), 0, s, t->view, keys, n);
  HKV_HIP(hipGetLastError());
  return HKV_SUCCESS;
}

int hkv_reserve(hkv_table* t, uint64_t new_capacity, hkv_stream_t stream) {
  HKV_TRY(refuse_dual(t, "reserve()", true));
  return reserve_impl(t, new_capacity, (hipStream_t)stream);
}

int hkv_set_max_capacity(hkv_table* t, uint64_t new_max_capacity) {
  if (!ispow2(new_max_capacity))
    return fail(HKV_ERROR_ARGUMENT, "None power-of-2 new_max_capacity is not supported.");
  if (new_max_capacity < t->view.capacity) return HKV_SUCCESS;
  t->reach_max_capacity = false;
  t->opts.max_capacity = new_max_capacity;
  return HKV_SUCCESS;
}

int hkv_clear(hkv_table* t, hkv_stream_t stream) {
  hipStream_t s = (hipStream_t)stream;
  LockGuard g(t, StreamGroupLock::kInserter, s);
  HKV_HIP(g.acquire());
  /* every key word becomes EMPTY, the LOCKED ones included */
  t->keys_may_be_locked = false;
  t->locked_recount = false;
  t->keys_offered = 0;
  t->bounds_stale = true;
  hipLaunchKernelGGL(zero_locked_kernel, dim3(1), dim3(kLockedShards), 0, s, t->d_locked);
  const uint64_t groups = t->view.capacity / 16;
  hipLaunchKernelGGL(fill_kernel, dim3((unsigned)((groups + 255) / 256)), dim3(256), 0, s,
                     t->view, 0);
  HKV_HIP(hipGetLastError());
  return HKV_SUCCESS;
}

int hkv_export_batch_if(const hkv_table* t, int predicate, uint64_t pattern,
                        uint64_t threshold, uint64_t n, uint64_t offset,
                        uint64_t* d_counter, uint64_t* keys, void* values,
                        uint64_t* scores, hkv_stream_t stream) {
  hipStream_t s = (hipStream_t)stream;
  if (predicate < HKV_PRED_ALWAYS || predicate > HKV_PRED_KEY_HIGH16_EQ_AND_SCORE_LT)
    return fail(HKV_ERROR_ARGUMENT, "unknown predicate %d", predicate);
  LockGuard g(t, StreamGroupLock::kReader, s);
  HKV_HIP(g.acquire());
  /* merlin_hashtable.cuh:3205-3213 */
  hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(1), 0, s, (unsigned long long*)d_counter);
  if (offset >= t->view.capacity) return HKV_SUCCESS;
  n = std::min(t->view.capacity - offset, n);
  if (n == 0) return HKV_SUCCESS;
  switch (predicate) {
    case HKV_PRED_ALWAYS:
      launch_export<PredAlways>(t, pattern, threshold, n, offset, d_counter, keys, values, scores, s);
      break;
    case HKV_PRED_SCORE_LT:
      launch_export<PredScoreLt>(t, pattern, threshold, n, offset, d_counter, keys, values, scores, s);
      break;
    case HKV_PRED_SCORE_LE:
      launch_export<PredScoreLe>(t, pattern, threshold, n, offset, d_counter, keys, values, scores, s);
      break;
    case HKV_PRED_SCORE_GT:
      launch_export<PredScoreGt>(t, pattern, threshold, n, offset, d_counter, keys, values, scores, s);
      break;
    case HKV_PRED_SCORE_GE:
      launch_export<PredScoreGe>(t, pattern, threshold, n, offset, d_counter, keys, values, scores, s);
      break;
    default:
      launch_export<PredKeyHigh16AndScoreLt>(t, pattern, threshold, n, offset, d_counter, keys, values, scores, s);
      break;
  }
  HKV_HIP(hipGetLastError());
  return HKV_SUCCESS;
}

int hkv_export_batch(const hkv_table* t, uint64_t n, uint64_t offset,
                     uint64_t* d_counter, uint64_t* keys, void* values,
                     uint64_t* scores, hkv_stream_t stream) {
  return hkv_export_batch_if(t, HKV_PRED_ALWAYS, 0, 0, n, offset, d_counter, keys,
                             values, scores, stream);
}

int hkv_size_if(const hkv_table* t, int predicate, uint64_t pattern,
                uint64_t threshold, hkv_stream_t stream, uint64_t* out) {
  hipStream_t s = (hipStream_t)stream;
  if (predicate < HKV_PRED_ALWAYS || predicate > HKV_PRED_KEY_HIGH16_EQ_AND_SCORE_LT)
    return fail(HKV_ERROR_ARGUMENT, "unknown predicate %d", predicate);
  CounterLease lease(t, s);
  unsigned long long* d = lease.word();
  {
    LockGuard g(t, StreamGroupLock::kReader, s);
    HKV_HIP(g.acquire());
    hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(1), 0, s, d);
    switch (predicate) {
      case HKV_PRED_ALWAYS: launch_size_if<PredAlways>(t, pattern, threshold, d, s); break;
      case HKV_PRED_SCORE_LT: launch_size_if<PredScoreLt>(t, pattern, threshold, d, s); break;
      case HKV_PRED_SCORE_LE: launch_size_if<PredScoreLe>(t, pattern, threshold, d, s); break;
      case HKV_PRED_SCORE_GT: launch_size_if<PredScoreGt>(t, pattern, threshold, d, s); break;
      case HKV_PRED_SCORE_GE: launch_size_if<PredScoreGe>(t, pattern, threshold, d, s); break;
      default: launch_size_if<PredKeyHigh16AndScoreLt>(t, pattern, threshold, d, s); break;
    }
    HKV_HIP(hipGetLastError());
  }
  return lease.read(out);
}

int hkv_size(const hkv_table* t, hkv_stream_t stream, uint64_t* out) {
  hipStream_t s = (hipStream_t)stream;
  CounterLease lease(t, s);
  unsigned long long* d = lease.word();
  {
    LockGuard g(t, StreamGroupLock::kReader, s);
    HKV_HIP(g.acquire());
    hipLaunchKernelGGL(zero_u64_kernel, dim3(1), dim3(1), 0, s, d);
    /* 16 digest bytes per lane and step; a workgroup per 2^16 slots, 512 at most */
    const unsigned blocks =
        (unsigned)std::min<uint64_t>((t->view.capacity + 65535) / 65536, 512);
    hipLaunchKernelGGL(size_kernel, dim3(blocks), dim3(256), 0, s, t->view, t->view.buckets_num, d);
    HKV_HIP(hipGetLastError());
  }
  return lease.read(out);
}

int hkv_empty(const hkv_table* t, hkv_stream_t stream, int* out) {
  uint64_t n = 0;
  HKV_TRY(hkv_size(t, stream, &n));
  *out = n == 0;
  return HKV_SUCCESS;
}

uint64_t hkv_capacity(const hkv_table* t) { return t->view.capacity; }

int hkv_load_factor(const hkv_table* t, hkv_stream_t stream, float* out) {
  uint64_t n = 0;
  HKV_TRY(hkv_size(t, stream, &n));
  *out = (float)((double)n / (double)t->view.capacity);
  return HKV_SUCCESS;
}

uint64_t hkv_dim(const hkv_table* t) { return t->opts.dim; }
uint64_t hkv_max_bucket_size(const hkv_table* t) { return t->opts.max_bucket_size; }
uint64_t hkv_bucket_count(const hkv_table* t) { return t->view.buckets_num; }
int hkv_is_pure_hbm(const hkv_table* t) { return t->pure_hbm; }

int hkv_set_global_epoch(hkv_table* t, uint64_t epoch) {
  /* scores of an earlier epoch are below what the score bounds were made for */
  if (epoch < t->epoch && t->epoch != kIgnoredEpoch) t->bounds_stale = true;
  t->epoch = epoch;
  return HKV_SUCCESS;
}

int hkv_table_get_view(const hkv_table* t, hkv_table_view* out) {
  *out = t->view;
  return HKV_SUCCESS;
}

int hkv_lock_begin(const hkv_table* t, int role, hkv_stream_t stream) {
  if (role < 0 || role > 2) return fail(HKV_ERROR_ARGUMENT, "bad lock role %d", role);
  if (!t->opts.api_lock) return HKV_SUCCESS;
  HKV_HIP(t->lock.begin((StreamGroupLock::Role)role, (hipStream_t)stream));
  return HKV_SUCCESS;
}

int hkv_lock_end(const hkv_table* t, int role, hkv_stream_t stream) {
  if (role < 0 || role > 2) return fail(HKV_ERROR_ARGUMENT, "bad lock role %d", role);
  if (!t->opts.api_lock) return HKV_SUCCESS;
  HKV_HIP(t->lock.end((StreamGroupLock::Role)role, (hipStream_t)stream));
  return HKV_SUCCESS;
}

int hkv_set_clock(hkv_table* t, int mode, uint64_t base) {
  if (mode != 0 && mode != 1) return fail(HKV_ERROR_ARGUMENT, "bad clock mode %d", mode);
  t->clock.mode = (uint32_t)mode;
  t->clock.base = base;
  t->bounds_stale = true; /* the new clock may be behind the old one */
  return HKV_SUCCESS;
}

int hkv_time_next_kernel(void* start_event, void* stop_event) {
  if ((start_event == nullptr) != (stop_event == nullptr))
    return fail(HKV_ERROR_ARGUMENT, "hkv_time_next_kernel takes two events or none");
  g_time_start = (hipEvent_t)start_event;
  g_time_stop = (hipEvent_t)stop_event;
  return HKV_SUCCESS;
}

int hkv_scores_changed(hkv_table* t) {
  t->bounds_stale = true;
  return HKV_SUCCESS;
}

}  // extern "C"
