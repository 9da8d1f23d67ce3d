/*
 * Table maintenance kernels: initial fill, clear, erase, size, and the
 * built-in export predicates.
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
  __shared__ unsigned long long s_part[4];
  for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = local;
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned long long total = s_part[0] + s_part[1] + s_part[2] + s_part[3];
    if (total) atomicAdd(out, total);
  }
}

__global__ void zero_u64_kernel(unsigned long long* p) { *p = 0; }
__global__ void zero_i32_kernel(int32_t* p) { *p = 0; }

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
