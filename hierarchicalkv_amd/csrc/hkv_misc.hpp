/*
 * Table maintenance kernels: initial fill, clear, erase, size, the assign
 * family (update existing keys only) and the built-in export predicates.
 */
#ifndef HKV_MISC_HPP_
#define HKV_MISC_HPP_

#include "hkv_lookup.hpp"

namespace hkv {

/* initialize_buckets (core_kernels.cuh:169-292) and clear_kernel (:656-676) in
 * one grid-wide fill: key = EMPTY, digest = EMPTY marker, size = 0; scores are
 * zeroed only at creation (clear leaves scores and values as they are).
 * One thread per 16 slots. */
__global__ void __launch_bounds__(256)
fill_kernel(View v, int zero_scores) {
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t groups = v.capacity / 16;
  if (t < groups) {
    const uint32_t e4 = v.empty_digest * 0x01010101u;
    reinterpret_cast<uint4*>(v.digests)[t] = make_uint4(e4, e4, e4, e4);
    uint64_t* k = v.keys + t * 16;
#pragma unroll
    for (int q = 0; q < 16; q++) k[q] = v.empty_key;
    if (zero_scores) {
      uint64_t* s = v.scores + t * 16;
#pragma unroll
      for (int q = 0; q < 16; q++) s[q] = 0;
    }
  }
  if (t < v.buckets_num) v.sizes[t] = 0;
}

/* remove_kernel (core_kernels.cuh:679-741): tombstone the slot. */
__global__ void __launch_bounds__(kWave)
erase_kernel(View v, const uint64_t* keys, uint64_t n) {
  __shared__ KeyMeta s_meta[kWave];
  __shared__ int64_t s_slot[kWave];
  const int lane = threadIdx.x;
  const uint64_t i = (uint64_t)blockIdx.x * kWave + lane;
  const uint64_t key = stage_keys(v, keys, n, i, s_meta, s_slot, lane);
  __syncthreads();
  probe_wave<false>(v, s_meta, s_slot, nullptr, nullptr, lane);
  __syncthreads();
  const int64_t slot = s_slot[lane];
  uint64_t seen = key;
  if (slot >= 0 && cas_lock(v.keys + slot, seen, v.reclaim_key)) {
    v.digests[slot] = v.reclaim_digest;
    v.scores[slot] = 0;
    atomicSub(v.sizes + (slot >> 7), 1);
  }
}

/* Sum of the per-bucket sizes (SumOp over buckets_size, core_kernels.cuh:1395-1423) */
__global__ void __launch_bounds__(256)
size_kernel(View v, unsigned long long* out) {
  uint64_t local = 0;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t b = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
       b < v.buckets_num; b += stride)
    local += (uint64_t)v.sizes[b];
  for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off);
  if ((threadIdx.x & 63) == 0 && local) atomicAdd(out, (unsigned long long)local);
}

__global__ void zero_u64_kernel(unsigned long long* p) { *p = 0; }
__global__ void zero_i32_kernel(int32_t* p) { *p = 0; }

/* ---- assign family: update keys that are present, never insert -------------
 * update kernels (update.cuh, update_score.cuh, update_values.cuh); the score
 * rule is ScoreFunctor::update_without_missed (kernel_utils.cuh:304-321,
 * 373-392, 436-453, 519-557, 594-612).  Several updaters may run at once (the
 * group lock lets them), so the row is changed under the slot lock. */

struct AssignArgs {
  const uint64_t* keys;
  const uint8_t* values; /* null: scores only */
  const uint64_t* scores;
  uint64_t n;
  uint64_t epoch;
  Clock clock;
  int32_t touch_scores;
  int32_t strategy;
};

__device__ __forceinline__ void assign_score(const View& v, const AssignArgs& a,
                                             uint64_t slot, uint64_t i) {
  const int STRATEGY = a.strategy;
  uint64_t s;
  if (STRATEGY == HKV_LRU) {
    s = now_ns(a.clock, i);
  } else if (STRATEGY == HKV_LFU) {
    if (!a.scores) return;
    s = ld_u64(v.scores + slot) + a.scores[i];
  } else if (STRATEGY == HKV_EPOCH_LRU) {
    s = (a.epoch << 32) | ((now_ns(a.clock, i) >> 20) & kLow32);
  } else if (STRATEGY == HKV_EPOCH_LFU) {
    if (!a.scores) return;
    const uint64_t in = a.scores[i] & kLow32;
    s = ld_u64(v.scores + slot) & kLow32;
    if (kLow32 - s > in)
      s += (a.epoch << 32) | in;
    else
      s = (a.epoch << 32) | kLow32;
  } else {
    if (!a.scores) return;
    s = a.scores[i];
  }
  st_u64(v.scores + slot, s);
}

template <int VEC>
__global__ void __launch_bounds__(kWave)
assign_kernel(View v, AssignArgs a) {
  __shared__ KeyMeta s_meta[kWave];
  __shared__ int64_t s_slot[kWave];
  __shared__ uint8_t s_unsure[kWave];
  const int lane = threadIdx.x;
  const int tile = lane >> 3, j = lane & 7;
  const uint64_t base = (uint64_t)blockIdx.x * kWave;
  stage_keys(v, a.keys, a.n, base + lane, s_meta, s_slot, lane);
  s_unsure[lane] = 0;
  __syncthreads();
  probe_wave<true>(v, s_meta, s_slot, nullptr, s_unsure, lane);
  __syncthreads();
#pragma unroll 1
  for (int r = 0; r < kTile; r++) {
    const int kk = r * kTile + tile;
    const uint64_t i = base + kk;
    const KeyMeta m = s_meta[kk];
    const uint64_t key = m.key;
    int64_t slot = s_slot[kk];
    bool reprobe = slot < 0 && s_unsure[kk];
    bool pending = slot >= 0 || reprobe;
    while (true) {
      if (pending && reprobe) {
        uint32_t em_unused;
        slot = tile_reprobe(v, key, m.bkt, m.info & 0xFFu, tile, j, em_unused);
        if (slot == -2) {
          __builtin_amdgcn_s_sleep(2);
        } else {
          reprobe = false;
          pending = slot >= 0;
        }
      } else if (pending) {
        int ok = 0;
        if (j == 0) {
          uint64_t seen = key;
          if (cas_lock(v.keys + slot, seen, v.locked_key))
            ok = 1;
          else if (seen != v.locked_key)
            ok = -1;
        }
        ok = tile_bcast(ok, tile, 0);
        if (ok > 0) {
          if (a.touch_scores && j == 0) assign_score(v, a, (uint64_t)slot, i);
          if (a.values)
            tile_copy<VEC, true, false>(value_row(v, (uint64_t)slot),
                                        a.values + i * v.value_bytes, v.value_bytes, j);
          wait_stores();
          if (j == 0) st_unlock(v.keys + slot, key);
          pending = false;
        } else if (ok < 0) {
          reprobe = true; /* the slot changed hands: look again */
        } else {
          __builtin_amdgcn_s_sleep(2);
        }
      }
      if (__ballot(pending) == 0) break;
    }
  }
}

/* ---- built-in predicates (hkv_predicate) -------------------------------------- */

struct PredAlways {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t&,
                                             const uint64_t&, const uint64_t&) const {
    return true;
  }
};
struct PredScoreLt {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s < th;
  }
};
struct PredScoreLe {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s <= th;
  }
};
struct PredScoreGt {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s > th;
  }
};
struct PredScoreGe {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s >= th;
  }
};
struct PredKeyHigh16AndScoreLt {
  __device__ __forceinline__ bool operator()(const uint64_t& k, uint64_t& s,
                                             const uint64_t& pat,
                                             const uint64_t& th) const {
    return (k & UINT64_C(0xFFFF000000000000)) == pat && s < th;
  }
};

}  // namespace hkv
#endif
