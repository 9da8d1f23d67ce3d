/*
 * Device-side view of a table and the kernels that a caller may need to
 * instantiate on its own functor types (export_batch_if<Pred>, size_if<Pred>).
 * Compiled by hipcc for gfx950 only; wavefronts are 64 lanes wide.
 *
 * Layout (flat arenas, no per-bucket pointers; replaces the per-bucket
 * allocations of core_kernels.cuh:169-292):
 *   digests[b][128] u8   one 128-byte line per bucket
 *   keys[b][128]    u64
 *   scores[b][128]  u64
 *   sizes[b]        i32
 *   values          slot-major rows of value_bytes; slots below hbm_slots in
 *                   HBM, the rest in pinned host memory (hybrid mode)
 */
#ifndef HKV_DEVICE_HPP_
#define HKV_DEVICE_HPP_

#include <hip/hip_cooperative_groups.h>
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "hkv_c_api.h"

namespace hkv {

constexpr uint32_t kBucketSize = 128;
constexpr int kWave = 64;

/* Murmur3 finaliser; same function as Murmur3HashDevice, utils.cuh:137-145 */
__host__ __device__ __forceinline__ uint64_t fmix64(uint64_t k) {
  k ^= k >> 33;
  k *= UINT64_C(0xff51afd7ed558ccd);
  k ^= k >> 33;
  k *= UINT64_C(0xc4ceb9fe1a85ec53);
  k ^= k >> 33;
  return k;
}

/* IS_RESERVED_KEY, types.cuh:70-73 */
__host__ __device__ __forceinline__ bool is_reserved_key(
    const hkv_table_view& v, uint64_t k) {
  return (k & v.reserved_mask1) == v.reserved_mask2;
}

/* Address of the value row of a slot. */
__device__ __forceinline__ uint8_t* value_row(const hkv_table_view& v,
                                              uint64_t slot) {
  if (slot < v.hbm_slots) return v.values + slot * v.value_bytes;
  return v.host_values + (slot - v.hbm_slots) * v.value_bytes;
}

__device__ __forceinline__ int lane_id() {
  return __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
}

/*
 * Copy one row of `bytes` bytes with all 64 lanes of the calling wavefront.
 * 16-byte units when size and both addresses allow it, else 4- or 1-byte units.
 */
__device__ __forceinline__ void wave_copy_row(uint8_t* dst, const uint8_t* src,
                                              uint32_t bytes, int lane) {
  const uintptr_t mis = (uintptr_t)dst | (uintptr_t)src | bytes;
  if ((mis & 15) == 0) {
    for (uint32_t u = lane; u < bytes / 16; u += kWave)
      reinterpret_cast<uint4*>(dst)[u] = reinterpret_cast<const uint4*>(src)[u];
  } else if ((mis & 3) == 0) {
    for (uint32_t u = lane; u < bytes / 4; u += kWave)
      reinterpret_cast<uint32_t*>(dst)[u] =
          reinterpret_cast<const uint32_t*>(src)[u];
  } else {
    for (uint32_t u = lane; u < bytes; u += kWave) dst[u] = src[u];
  }
}

/*
 * export_batch_if: scan slots [offset, offset + n) in slot order, append every
 * entry whose key is not reserved and for which pred(key, score, pattern,
 * threshold) holds.  Output is compact and unordered across wavefronts
 * (same contract as dump_kernel_v2, core_kernels.cuh:983-1041).
 *
 * One slot per lane for the key / score scan; a 64-bit ballot gives the
 * wavefront's match set, one atomic per wavefront reserves the output range,
 * and the wavefront then copies the matched rows cooperatively.
 * `values` and `scores` may be null.
 */
template <class Pred>
__global__ void __launch_bounds__(256)
export_if_kernel(hkv_table_view v, Pred pred, uint64_t pattern,
                 uint64_t threshold, uint64_t offset, uint64_t n,
                 unsigned long long* counter, uint64_t* out_keys,
                 uint8_t* out_values, uint64_t* out_scores) {
  const int lane = lane_id();
  const uint64_t wave_global =
      ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  const uint64_t waves_total = ((uint64_t)gridDim.x * blockDim.x) / kWave;
  const uint64_t chunks = (n + kWave - 1) / kWave;
  for (uint64_t c = wave_global; c < chunks; c += waves_total) {
    const uint64_t i = c * kWave + lane;
    uint64_t slot = offset + i;
    uint64_t key = v.empty_key;
    uint64_t score = 0;
    bool match = false;
    if (i < n) {
      key = v.keys[slot];
      score = v.scores[slot];
      match = !is_reserved_key(v, key) && pred(key, score, pattern, threshold);
    }
    const unsigned long long vote = __ballot(match);
    if (vote == 0) continue;
    const int cnt = __popcll(vote);
    unsigned long long base = 0;
    if (lane == 0) base = atomicAdd(counter, (unsigned long long)cnt);
    base = __shfl(base, 0);
    const int rank = __popcll(vote & ((1ull << lane) - 1));
    if (match) {
      out_keys[base + rank] = key;
      if (out_scores) out_scores[base + rank] = score;
    }
    if (out_values) {
      unsigned long long rest = vote;
      int r = 0;
      while (rest) {
        const int src_lane = __ffsll(rest) - 1;
        rest &= rest - 1;
        const uint64_t s = offset + c * kWave + src_lane;
        wave_copy_row(out_values + (base + r) * v.value_bytes, value_row(v, s),
                      v.value_bytes, lane);
        r++;
      }
    }
  }
}

/* size_if: number of entries satisfying the predicate (size_if_kernel,
 * core_kernels.cuh:1114-1151). */
template <class Pred>
__global__ void __launch_bounds__(256)
size_if_kernel(hkv_table_view v, Pred pred, uint64_t pattern,
               uint64_t threshold, unsigned long long* counter) {
  const int lane = lane_id();
  uint64_t local = 0;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t s = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
       s < v.capacity; s += stride) {
    uint64_t key = v.keys[s];
    uint64_t score = v.scores[s];
    if (!is_reserved_key(v, key) && pred(key, score, pattern, threshold)) local++;
  }
  for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off);
  if (lane == 0 && local) atomicAdd(counter, (unsigned long long)local);
}

/* erase_if: tombstone every entry the predicate selects (the predicate form of
 * remove_kernel, core_kernels.cuh:744-843).  Runs under the inserter role, so
 * no other kernel touches the table meanwhile. */
template <class Pred>
__global__ void __launch_bounds__(256)
erase_if_kernel(hkv_table_view v, Pred pred, uint64_t pattern, uint64_t threshold,
                unsigned long long* counter) {
  const int lane = lane_id();
  uint64_t local = 0;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t s = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
       s < v.capacity; s += stride) {
    uint64_t key = v.keys[s];
    uint64_t score = v.scores[s];
    if (!is_reserved_key(v, key) && pred(key, score, pattern, threshold)) {
      v.keys[s] = v.reclaim_key;
      v.digests[s] = v.reclaim_digest;
      v.scores[s] = 0;
      atomicSub(v.sizes + (s >> 7), 1);
      local++;
    }
  }
  for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off);
  if (lane == 0 && local) atomicAdd(counter, (unsigned long long)local);
}

/*
 * Tile type handed to the functor forms below.  It is HIP's
 * cooperative_groups::thread_block_tile<N> plus shuffles of pointers, which
 * functors written for the reference use (g.shfl(value, r) on a row pointer,
 * tests/export_batch_if_test.cc.cu:117) and HIP's own tile does not take.
 * Everything else of cooperative_groups is visible through this namespace, so
 * it can stand behind a `cg` alias the way merlin/utils.cuh:30 sets one up.
 */
namespace coop {
using namespace cooperative_groups;

template <unsigned int N>
class thread_block_tile : public cooperative_groups::thread_block_tile<N> {
  using Base = cooperative_groups::thread_block_tile<N>;

 public:
  template <class Parent>
  __device__ thread_block_tile(const cooperative_groups::thread_block_tile<N, Parent>& t)
      : Base(t) {}

  template <class T>
  __device__ T shfl(T var, int src_rank) const {
    if constexpr (std::is_pointer<T>::value)
      return reinterpret_cast<T>(Base::shfl(reinterpret_cast<unsigned long long>(var), src_rank));
    else
      return Base::shfl(var, src_rank);
  }
  template <class T>
  __device__ T shfl_down(T var, unsigned int delta) const {
    if constexpr (std::is_pointer<T>::value)
      return reinterpret_cast<T>(Base::shfl_down(reinterpret_cast<unsigned long long>(var), delta));
    else
      return Base::shfl_down(var, delta);
  }
  template <class T>
  __device__ T shfl_up(T var, unsigned int delta) const {
    if constexpr (std::is_pointer<T>::value)
      return reinterpret_cast<T>(Base::shfl_up(reinterpret_cast<unsigned long long>(var), delta));
    else
      return Base::shfl_up(var, delta);
  }
  template <class T>
  __device__ T shfl_xor(T var, unsigned int mask) const {
    if constexpr (std::is_pointer<T>::value)
      return reinterpret_cast<T>(Base::shfl_xor(reinterpret_cast<unsigned long long>(var), mask));
    else
      return Base::shfl_xor(var, mask);
  }
};
}  // namespace coop

/*
 * The functor forms that see the value row and work in cooperative-groups
 * tiles: f.template operator()<GroupSize>(key, value, score, tile).  The tile
 * is hkv::coop::thread_block_tile<GroupSize>; the caller picks
 * GroupSize so that the slot count is a multiple of it (all threads of a tile
 * take the same number of trips).  K, V, S are the caller's types over the
 * table's 64-bit key / score words and value bytes.
 *
 * traverse_kernel, core_kernels.cuh:1153-1178 (for_each)
 */
template <class K, class V, class S, class Func, unsigned GroupSize>
__global__ void __launch_bounds__(128)
traverse_kernel(hkv_table_view v, uint64_t n, uint64_t offset, Func f) {
  coop::thread_block_tile<GroupSize> g(coop::tiled_partition<GroupSize>(coop::this_thread_block()));
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint64_t slot = i + offset;
    const K key = static_cast<K>(v.keys[slot]);
    S* score = reinterpret_cast<S*>(v.scores + slot);
    V* value = reinterpret_cast<V*>(value_row(v, slot));
    f.template operator()<GroupSize>(key, value, score, g);
  }
}

/* dump_kernel with a functor, core_kernels.cuh:1043-1112 (export_batch_if_v2):
 * the functor alone decides, reserved keys included */
template <class K, class V, class S, class Pred, unsigned GroupSize>
__global__ void __launch_bounds__(128)
export_if_v2_kernel(hkv_table_view v, uint64_t n, uint64_t offset, Pred pred,
                    unsigned long long* counter, K* out_keys, V* out_values, S* out_scores) {
  coop::thread_block_tile<GroupSize> g(coop::tiled_partition<GroupSize>(coop::this_thread_block()));
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  const uint32_t dim = v.value_bytes / sizeof(V);
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    const uint64_t slot = i + offset;
    const K key = static_cast<K>(v.keys[slot]);
    const S score = static_cast<S>(v.scores[slot]);
    const V* value = reinterpret_cast<const V*>(value_row(v, slot));
    const bool match = pred.template operator()<GroupSize>(key, value, score, g);
    const unsigned long long vote = g.ballot(match);
    const int cnt = __popcll(vote);
    unsigned long long base = 0;
    if (g.thread_rank() == 0 && cnt) base = atomicAdd(counter, (unsigned long long)cnt);
    base = g.shfl(base, 0);
    const int before = __popcll(vote & ((1ull << g.thread_rank()) - 1));
    if (match) {
      out_keys[base + before] = key;
      if (out_scores) out_scores[base + before] = score;
    }
    for (unsigned r = 0; r < GroupSize; r++) {
      if (!((vote >> r) & 1ull)) continue;
      const int bias = __popcll(vote & ((1ull << r) - 1));
      const uint64_t cur = (i / GroupSize) * GroupSize + r + offset;
      const V* src = reinterpret_cast<const V*>(value_row(v, cur));
      for (uint32_t d = g.thread_rank(); d < dim; d += GroupSize)
        out_values[(base + bias) * dim + d] = src[d];
    }
  }
}

/* remove_kernel_v2, core_kernels.cuh:794-843 (erase_if_v2) */
template <class K, class V, class S, class Pred, unsigned GroupSize>
__global__ void __launch_bounds__(128)
erase_if_v2_kernel(hkv_table_view v, uint64_t n, Pred pred, unsigned long long* counter) {
  coop::thread_block_tile<GroupSize> g(coop::tiled_partition<GroupSize>(coop::this_thread_block()));
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t slot = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; slot < n; slot += stride) {
    const uint64_t raw = v.keys[slot];
    const K key = static_cast<K>(raw);
    const S score = static_cast<S>(v.scores[slot]);
    const V* value = reinterpret_cast<const V*>(value_row(v, slot));
    bool match = pred.template operator()<GroupSize>(key, value, score, g);
    if (is_reserved_key(v, raw)) match = false;
    const unsigned long long vote = g.ballot(match);
    const int cnt = __popcll(vote);
    /* GroupSize divides 128, so the slots of a tile share a bucket */
    if (g.thread_rank() == 0 && cnt) {
      atomicAdd(counter, (unsigned long long)cnt);
      atomicSub(v.sizes + (slot >> 7), cnt);
    }
    if (match) {
      v.digests[slot] = v.reclaim_digest;
      v.keys[slot] = v.reclaim_key;
      v.scores[slot] = 0;
    }
  }
}

/* One-word clear as a kernel: callers may be capturing a graph, where memset
 * nodes are best avoided. */
template <class T>
__global__ void zero_word_kernel(T* p) {
  *p = T(0);
}

}  // namespace hkv
#endif
