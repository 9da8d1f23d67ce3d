/*
 * lock_keys / unlock_keys / find_and_update: the calls that hand out addresses
 * of key words and value rows together with a score touch.
 *
 * Replaces lock_kernel_with_filter and unlock_keys_kernel
 * (core_kernels.cuh:1180-1204, 1248-1362) and the update_score = true form of
 * tlp_lookup_ptr_kernel_with_filter (lookup_ptr.cuh:25-150).  One wavefront per
 * 64 keys, probe as in find.
 */
#ifndef HKV_KEYLOCKS_HPP_
#define HKV_KEYLOCKS_HPP_

#include "hkv_grouped.hpp"

namespace hkv {

struct TouchArgs {
  const uint64_t* keys;
  uint64_t* scores;      /* input of the score rule; find_and_update also writes the result back */
  uint64_t** key_ptrs;   /* lock_keys */
  void** value_ptrs;     /* find_and_update */
  uint8_t* flags;        /* success / founds, may be null */
  unsigned long long* locked_count; /* lock_keys: the table's count of slots left LOCKED */
  uint64_t n;
  uint64_t epoch;
  Clock clock;
  int32_t strategy;
};

/* the score a key that is present gets from an upsert-family call
 * (update_with_digest with is_insert = false); the caller holds the slot */
__device__ __forceinline__ uint64_t touch_score(const View& v, const TouchArgs& t, int64_t slot,
                                                uint64_t i) {
  UpsertArgs a{};
  a.scores = t.scores;
  a.epoch = t.epoch;
  a.clock = t.clock;
  a.strategy = t.strategy;
  const uint64_t in_score = t.scores ? t.scores[i] : 0;
  const uint64_t desired = desired_when_missed(a, in_score, i);
  const bool needs_old = t.strategy == HKV_LFU || t.strategy == HKV_EPOCH_LFU;
  /* the old score is only read where the new one is made from it (a line of memory traffic
   * per key otherwise) */
  const uint64_t old = needs_old ? ld_u64(v.scores + slot) : 0;
  uint64_t snew;
  if (!final_score(a, false, desired, in_score, old, snew)) return ld_u64(v.scores + slot);
  st_u64(v.scores + slot, snew);
  return snew;
}

/* KEEP_LOCKED: lock_keys (the key word stays LOCKED, its address goes out);
 * otherwise find_and_update (lock, touch, unlock; row address and score out) */
template <bool KEEP_LOCKED>
__global__ void __launch_bounds__(kWave)
touch_kernel(View v, TouchArgs t) {
  __shared__ KeyMeta s_meta[kWave];
  __shared__ int64_t s_slot[kWave];
  const int lane = threadIdx.x;
  const uint64_t i = (uint64_t)blockIdx.x * kWave + lane;
  const uint64_t key = stage_keys(v, t.keys, t.n, i, s_meta, s_slot, lane);
  __syncthreads();
  probe_wave<false, false>(v, s_meta, s_slot, nullptr, nullptr, lane);
  __syncthreads();
  const int64_t slot = s_slot[lane];
  bool ok = false;
  uint64_t score = 0;
  if (i < t.n && slot >= 0) {
    /* several updaters may run at once: the slot lock is taken as everywhere */
    uint64_t seen = key;
    for (int tries = 0; tries < kMaxLockedWaits && !ok; tries++) {
      seen = key;
      ok = cas_lock(v.keys + slot, seen, v.locked_key);
      if (!ok && seen != v.locked_key) break; /* the slot changed hands */
      if (!ok) __builtin_amdgcn_s_sleep(2);
    }
    if (ok) {
      score = touch_score(v, t, slot, i);
      if (!KEEP_LOCKED) {
        wait_stores();
        st_unlock(v.keys + slot, key);
      }
    }
  }
  if (KEEP_LOCKED) {
    /* one update of the table's count per wavefront */
    const unsigned long long kept = __ballot(ok);
    if (kept && lane == (int)__ffsll(kept) - 1)
      atomicAdd(locked_shard(t.locked_count), (unsigned long long)__popcll(kept));
  }
  if (i >= t.n) return;
  if (t.flags) t.flags[i] = ok;
  if (KEEP_LOCKED) {
    t.key_ptrs[i] = ok ? v.keys + slot : nullptr;
  } else {
    t.value_ptrs[i] = ok ? value_row(v, (uint64_t)slot) : nullptr;
    if (ok && t.scores) t.scores[i] = score;
  }
}

/* unlock_keys_kernel, core_kernels.cuh:1180-1204 */
__global__ void __launch_bounds__(256)
unlock_keys_kernel(View v, uint64_t n, uint64_t* const* key_ptrs, const uint64_t* keys,
                   uint8_t* success, unsigned long long* locked_count) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t* p = i < n ? key_ptrs[i] : nullptr;
  bool ok = false;
  if (p != nullptr && ld_u64(p) == v.locked_key) {
    st_u64(p, keys[i]);
    ok = true;
  }
  const unsigned long long freed = __ballot(ok);
  if (locked_count && freed && (threadIdx.x & (kWave - 1)) == (int)__ffsll(freed) - 1)
    atomicAdd(locked_shard(locked_count), 0ull - (unsigned long long)__popcll(freed)) /* wraps: a subtraction */;
  if (i < n && success) success[i] = ok;
}

/* The second launch of an upsert in hybrid mode: every slot the first one left LOCKED gets its
 * score (it showed kMaxScore meanwhile, so that no key of the batch took it for a victim) and then
 * its key.  The caller has the table to itself. */
__global__ void __launch_bounds__(256)
open_held_kernel(View v, uint64_t n, uint64_t* const* key_ptrs, const uint64_t* scores, const uint64_t* keys) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  uint64_t* p = i < n ? key_ptrs[i] : nullptr;
  if (p != nullptr) {
    const uint64_t s = scores[i];
    if (s != kMaxScore) st_u64(v.scores + (p - v.keys), s);
  }
  wait_stores();
  if (p != nullptr) st_u64(p, keys[i]);
}

}  // namespace hkv
#endif
