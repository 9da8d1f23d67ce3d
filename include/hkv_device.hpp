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
 *   sizes[b]        i32  keys per bucket, dual-bucket tables only (elsewhere a slot holds a key
 *                        exactly when its digest is not the EMPTY marker)
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

/* ---- compaction shared by the export kernels ---------------------------------------------
 *
 * A workgroup scans a chunk of slots, every thread keeping up to kExportPerThread
 * matches in registers.  The matches of the chunk get consecutive output positions from
 * ONE atomic on the caller's counter per chunk (atomics on one word serialise on this
 * memory system, about 15 ns each: one per wavefront made the counter the bottleneck of
 * the whole export), and the rows are then copied by the whole workgroup from a list of
 * matched slots in LDS, with streaming loads and stores.  Output order is unspecified,
 * as with dump_kernel_v2 (core_kernels.cuh:983-1041).
 */
constexpr int kExportPerThread = 8;

/* exclusive position of this thread's `cnt` matches inside the workgroup's chunk, and the
 * chunk's total; all threads of the workgroup call it (two barriers) */
template <int THREADS>
__device__ __forceinline__ uint32_t block_offsets(uint32_t cnt, uint32_t* s_wave, uint32_t& total) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  uint32_t inc = cnt;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const uint32_t t = __shfl_up(inc, off);
    if (lane >= off) inc += t;
  }
  __syncthreads(); /* s_wave of the previous chunk has been read by everybody */
  if (lane == kWave - 1) s_wave[wave] = inc;
  __syncthreads();
  uint32_t before = 0;
  total = 0;
#pragma unroll
  for (int w = 0; w < THREADS / kWave; w++) {
    const uint32_t t = s_wave[w];
    if (w < wave) before += t;
    total += t;
  }
  return before + inc - cnt;
}

/* rows of the chunk's matches: s_src[r] is the slot (relative to `first_slot`) of match r,
 * which goes to output row `base + r`; UNIT bytes per thread and trip, 4 trips in flight */
template <int THREADS, class T>
__device__ __forceinline__ void export_rows(const hkv_table_view& v, uint64_t first_slot,
                                            const uint16_t* s_src, uint32_t total,
                                            unsigned long long base, uint8_t* out_values) {
  const uint32_t units = v.value_bytes / sizeof(T);
  const uint32_t tu = total * units;
  constexpr int kBatch = 4;
  for (uint32_t idx0 = threadIdx.x; idx0 < tu; idx0 += THREADS * kBatch) {
    T buf[kBatch];
    uint32_t row[kBatch], cc[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; b++) {
      const uint32_t idx = idx0 + b * THREADS;
      row[b] = idx / units;
      cc[b] = idx - row[b] * units;
      if (idx < tu)
        buf[b] = __builtin_nontemporal_load(
            reinterpret_cast<const T*>(value_row(v, first_slot + s_src[row[b]])) + cc[b]);
    }
#pragma unroll
    for (int b = 0; b < kBatch; b++) {
      const uint32_t idx = idx0 + b * THREADS;
      if (idx < tu)
        __builtin_nontemporal_store(
            buf[b], reinterpret_cast<T*>(out_values + (base + row[b]) * v.value_bytes) + cc[b]);
    }
  }
}
template <int THREADS>
__device__ __forceinline__ void export_rows_any(const hkv_table_view& v, uint64_t first_slot,
                                                const uint16_t* s_src, uint32_t total,
                                                unsigned long long base, uint8_t* out_values) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const uintptr_t mis = (uintptr_t)out_values | v.value_bytes;
  if ((mis & 15) == 0)
    export_rows<THREADS, u32x4_t>(v, first_slot, s_src, total, base, out_values);
  else if ((mis & 3) == 0)
    export_rows<THREADS, uint32_t>(v, first_slot, s_src, total, base, out_values);
  else
    export_rows<THREADS, uint8_t>(v, first_slot, s_src, total, base, out_values);
}

/*
 * export_batch_if: scan slots [offset, offset + n), append every entry whose key is not
 * reserved and for which pred(key, score, pattern, threshold) holds.  `values` and
 * `scores` may be null.
 */
constexpr int kExportThreads = 256;
template <class Pred>
__global__ void __launch_bounds__(kExportThreads)
export_if_kernel(hkv_table_view v, Pred pred, uint64_t pattern,
                 uint64_t threshold, uint64_t offset, uint64_t n,
                 unsigned long long* counter, uint64_t* out_keys,
                 uint8_t* out_values, uint64_t* out_scores) {
  constexpr int kChunk = kExportThreads * kExportPerThread;
  __shared__ uint16_t s_src[kChunk];
  __shared__ uint32_t s_wave[kExportThreads / kWave];
  __shared__ unsigned long long s_base;
  const int tid = threadIdx.x;
  const uint64_t chunks = (n + kChunk - 1) / kChunk;
  for (uint64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
    const uint64_t cbase = c * kChunk;
    uint64_t key[kExportPerThread], score[kExportPerThread];
#pragma unroll
    for (int r = 0; r < kExportPerThread; r++) {
      const uint64_t i = cbase + (uint64_t)r * kExportThreads + tid;
      key[r] = v.empty_key;
      score[r] = 0;
      if (i < n) {
        key[r] = v.keys[offset + i];
        score[r] = v.scores[offset + i];
      }
    }
    uint32_t mask = 0;
#pragma unroll
    for (int r = 0; r < kExportPerThread; r++)
      if (!is_reserved_key(v, key[r]) && pred(key[r], score[r], pattern, threshold)) mask |= 1u << r;
    uint32_t total;
    uint32_t at = block_offsets<kExportThreads>((uint32_t)__popc(mask), s_wave, total);
    if (total == 0) continue; /* the same for the whole workgroup */
    if (tid == 0) s_base = atomicAdd(counter, (unsigned long long)total);
    {
      uint32_t a = at;
#pragma unroll
      for (int r = 0; r < kExportPerThread; r++)
        if (mask & (1u << r)) s_src[a++] = (uint16_t)(r * kExportThreads + tid);
    }
    __syncthreads();
    const unsigned long long base = s_base;
#pragma unroll
    for (int r = 0; r < kExportPerThread; r++) {
      if (mask & (1u << r)) {
        out_keys[base + at] = key[r];
        if (out_scores) out_scores[base + at] = score[r];
        at++;
      }
    }
    if (out_values) export_rows_any<kExportThreads>(v, offset + cbase, s_src, total, base, out_values);
    __syncthreads(); /* s_src and s_base are reused by the next chunk */
  }
}

/* sum of `local` over the workgroup, one atomic per workgroup */
__device__ __forceinline__ void block_count(uint64_t local, unsigned long long* counter) {
  __shared__ unsigned long long s_sum;
  if (threadIdx.x == 0) s_sum = 0;
  __syncthreads();
  for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off);
  if (lane_id() == 0 && local) atomicAdd(&s_sum, (unsigned long long)local);
  __syncthreads();
  if (threadIdx.x == 0 && s_sum) atomicAdd(counter, s_sum);
}

/* size_if: number of entries satisfying the predicate (size_if_kernel,
 * core_kernels.cuh:1114-1151). */
template <class Pred>
__global__ void __launch_bounds__(256)
size_if_kernel(hkv_table_view v, Pred pred, uint64_t pattern,
               uint64_t threshold, unsigned long long* counter) {
  uint64_t local = 0;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t s = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
       s < v.capacity; s += stride) {
    uint64_t key = v.keys[s];
    uint64_t score = v.scores[s];
    if (!is_reserved_key(v, key) && pred(key, score, pattern, threshold)) local++;
  }
  block_count(local, counter);
}

/* erase_if: tombstone every entry the predicate selects (the predicate form of
 * remove_kernel, core_kernels.cuh:744-843).  Runs under the inserter role, so
 * no other kernel touches the table meanwhile. */
template <class Pred>
__global__ void __launch_bounds__(256)
erase_if_kernel(hkv_table_view v, Pred pred, uint64_t pattern, uint64_t threshold,
                unsigned long long* counter) {
  uint64_t local = 0;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t s = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
       s < v.capacity; s += stride) {
    uint64_t key = v.keys[s];
    uint64_t score = v.scores[s];
    if (!is_reserved_key(v, key) && pred(key, score, pattern, threshold)) {
      /* a free slot again, not a tombstone: see erase_kernel */
      v.keys[s] = v.empty_key;
      v.digests[s] = v.empty_digest;
      if (v.sizes) atomicSub(v.sizes + (s >> 7), 1);
      local++;
    }
  }
  block_count(local, counter);
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
 * the functor alone decides, reserved keys included.  The tiles evaluate the functor slot
 * by slot; the matches of a chunk are then compacted as in export_if_kernel. */
constexpr int kExportV2Threads = 128;
template <class K, class V, class S, class Pred, unsigned GroupSize>
__global__ void __launch_bounds__(kExportV2Threads)
export_if_v2_kernel(hkv_table_view v, uint64_t n, uint64_t offset, Pred pred,
                    unsigned long long* counter, K* out_keys, V* out_values, S* out_scores) {
  constexpr int kChunk = kExportV2Threads * kExportPerThread;
  __shared__ uint16_t s_src[kChunk];
  __shared__ uint32_t s_wave[kExportV2Threads / kWave];
  __shared__ unsigned long long s_base;
  coop::thread_block_tile<GroupSize> g(coop::tiled_partition<GroupSize>(coop::this_thread_block()));
  const int tid = threadIdx.x;
  const uint64_t chunks = (n + kChunk - 1) / kChunk;
  for (uint64_t c = blockIdx.x; c < chunks; c += gridDim.x) {
    const uint64_t cbase = c * kChunk;
    uint64_t key[kExportPerThread], score[kExportPerThread];
    uint32_t mask = 0;
#pragma unroll
    for (int r = 0; r < kExportPerThread; r++) {
      const uint64_t i = cbase + (uint64_t)r * kExportV2Threads + tid;
      key[r] = 0;
      score[r] = 0;
      /* the caller picks GroupSize so that n is a multiple of it: a tile is inside or outside */
      if (i < n) {
        const uint64_t slot = offset + i;
        key[r] = v.keys[slot];
        score[r] = v.scores[slot];
        const V* value = reinterpret_cast<const V*>(value_row(v, slot));
        if (pred.template operator()<GroupSize>(static_cast<K>(key[r]), value,
                                                static_cast<S>(score[r]), g))
          mask |= 1u << r;
      }
    }
    uint32_t total;
    uint32_t at = block_offsets<kExportV2Threads>((uint32_t)__popc(mask), s_wave, total);
    if (total == 0) continue;
    if (tid == 0) s_base = atomicAdd(counter, (unsigned long long)total);
    {
      uint32_t a = at;
#pragma unroll
      for (int r = 0; r < kExportPerThread; r++)
        if (mask & (1u << r)) s_src[a++] = (uint16_t)(r * kExportV2Threads + tid);
    }
    __syncthreads();
    const unsigned long long base = s_base;
#pragma unroll
    for (int r = 0; r < kExportPerThread; r++) {
      if (mask & (1u << r)) {
        out_keys[base + at] = static_cast<K>(key[r]);
        if (out_scores) out_scores[base + at] = static_cast<S>(score[r]);
        at++;
      }
    }
    export_rows_any<kExportV2Threads>(v, offset + cbase, s_src, total, base,
                                      reinterpret_cast<uint8_t*>(out_values));
    __syncthreads();
  }
}

/* remove_kernel_v2, core_kernels.cuh:794-843 (erase_if_v2) */
template <class K, class V, class S, class Pred, unsigned GroupSize>
__global__ void __launch_bounds__(128)
erase_if_v2_kernel(hkv_table_view v, uint64_t n, Pred pred, unsigned long long* counter) {
  coop::thread_block_tile<GroupSize> g(coop::tiled_partition<GroupSize>(coop::this_thread_block()));
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  uint64_t local = 0;
  for (uint64_t slot = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; slot < n; slot += stride) {
    const uint64_t raw = v.keys[slot];
    const K key = static_cast<K>(raw);
    const S score = static_cast<S>(v.scores[slot]);
    const V* value = reinterpret_cast<const V*>(value_row(v, slot));
    bool match = pred.template operator()<GroupSize>(key, value, score, g);
    if (is_reserved_key(v, raw)) match = false;
    if (match) {
      v.digests[slot] = v.empty_digest;
      v.keys[slot] = v.empty_key;
      if (v.sizes) atomicSub(v.sizes + (slot >> 7), 1);
      local++;
    }
  }
  block_count(local, counter);
}

/* launch shapes of the scans above */
inline unsigned export_grid(uint64_t n, int threads) {
  const uint64_t chunks = (n + (uint64_t)threads * kExportPerThread - 1) / ((uint64_t)threads * kExportPerThread);
  return (unsigned)(chunks < 4096 ? (chunks ? chunks : 1) : 4096);
}
inline unsigned scan_grid(uint64_t slots, int threads) {
  const uint64_t blocks = (slots + threads - 1) / threads;
  return (unsigned)(blocks < 2048 ? (blocks ? blocks : 1) : 2048);
}

/* 32-bit score arrays of the caller <-> the table's 64-bit scores (zero-extended) */
__global__ void widen_scores_kernel(const uint32_t* in, uint64_t* out, uint64_t n) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = in[i];
}
__global__ void narrow_scores_kernel(const uint64_t* in, uint32_t* out, uint64_t n) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = (uint32_t)in[i];
}

/* One-word clear as a kernel: callers may be capturing a graph, where memset
 * nodes are best avoided. */
template <class T>
__global__ void zero_word_kernel(T* p) {
  *p = T(0);
}

}  // namespace hkv
#endif
