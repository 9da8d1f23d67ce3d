/*
 * Batches that may hold a key more than once (unique_key = false).
 *
 * The reference switches to its lock-per-bucket kernels for such batches
 * (merlin_hashtable.cuh:1194-1252, 1737-1790, 1925-1960): every occurrence is applied,
 * in no particular order, and the table ends up holding the key once (tests/
 * find_or_insert_ptr_test.cc.cu:3390-3475: 1024 copies of one key leave one entry).  Here
 * the batch is reduced to one occurrence per key before the ordinary kernels run: a stable
 * radix sort of (key, index) finds the runs of equal keys, the first occurrence of a run
 * stands for the key, and the other occurrences travel as the EMPTY key, which every
 * kernel skips.  Calls that hand something back per key (find_or_insert) copy it from the
 * representative afterwards.
 */
#ifndef HKV_DEDUP_HPP_
#define HKV_DEDUP_HPP_

#include <hipcub/hipcub.hpp>

#include "hkv_common.hpp"

namespace hkv {

struct DedupPlan {
  uint64_t* keys = nullptr; /* [n] the batch with later occurrences replaced by EMPTY */
  uint32_t* rep = nullptr;  /* [n] index of the occurrence that stands for key i */
  void* block = nullptr;
  hipStream_t stream = nullptr;
};

__global__ void dedup_init_kernel(const uint64_t* keys, uint64_t* keys_mod, uint32_t* idx, uint64_t n) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) {
    keys_mod[i] = keys[i];
    idx[i] = (uint32_t)i;
  }
}
/* head[p] = p where a run of equal keys starts, else 0 (a running maximum then gives the
 * start of the run every position belongs to) */
__global__ void dedup_heads_kernel(const uint64_t* skeys, uint32_t* head, uint64_t n) {
  const uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p < n) head[p] = (p == 0 || skeys[p - 1] != skeys[p]) ? (uint32_t)p : 0u;
}
__global__ void dedup_mark_kernel(const uint32_t* sidx, const uint32_t* start, uint64_t n,
                                  uint64_t empty_key, uint64_t* keys_mod, uint32_t* rep) {
  const uint64_t p = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= n) return;
  const uint32_t i = sidx[p];
  const uint32_t first = start[p];
  rep[i] = sidx[first];
  if (first != (uint32_t)p) keys_mod[i] = empty_key;
}
/* what a duplicate gets back: the representative's pointer and flag ... */
__global__ void dedup_fix_ptrs_kernel(const uint32_t* rep, uint64_t n, void** out_ptrs, uint8_t* founds) {
  const uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const uint32_t r = rep[i];
  if (r == (uint32_t)i) return;
  if (out_ptrs) out_ptrs[i] = out_ptrs[r];
  if (founds) founds[i] = founds[r];
}
/* ... or its row (4 bytes per thread and trip when the row allows it, else single bytes) */
__global__ void dedup_fix_rows_kernel(const uint32_t* rep, uint64_t n, uint8_t* rows, uint32_t row_bytes) {
  const uint64_t i = blockIdx.x;
  if (i >= n) return;
  const uint32_t r = rep[i];
  if (r == (uint32_t)i) return;
  uint8_t* dst = rows + i * (uint64_t)row_bytes;
  const uint8_t* src = rows + r * (uint64_t)row_bytes;
  if (((row_bytes | (uintptr_t)rows) & 3) == 0) {
    for (uint32_t u = threadIdx.x; u < row_bytes / 4; u += blockDim.x)
      reinterpret_cast<uint32_t*>(dst)[u] = reinterpret_cast<const uint32_t*>(src)[u];
  } else {
    for (uint32_t u = threadIdx.x; u < row_bytes; u += blockDim.x) dst[u] = src[u];
  }
}

struct MaxU32 {
  __host__ __device__ uint32_t operator()(uint32_t a, uint32_t b) const { return a > b ? a : b; }
};

inline void dedup_free(DedupPlan& d) {
  if (d.block) (void)hipFreeAsync(d.block, d.stream);
  d.block = nullptr;
}

/* Builds d.keys and d.rep for the n keys of a batch on stream s (n < 2^32). */
inline hipError_t dedup_make(const View& v, uint64_t n, const uint64_t* keys, hipStream_t s,
                             DedupPlan& d) {
  d.stream = s;
  auto up = [](uint64_t x) { return (x + 255) & ~UINT64_C(255); };
  size_t sort_bytes = 0, scan_bytes = 0;
  hipError_t e = hipcub::DeviceRadixSort::SortPairs(
      nullptr, sort_bytes, (const uint64_t*)nullptr, (uint64_t*)nullptr, (const uint32_t*)nullptr,
      (uint32_t*)nullptr, (int)n, 0, 64, s);
  if (e != hipSuccess) return e;
  e = hipcub::DeviceScan::InclusiveScan(nullptr, scan_bytes, (const uint32_t*)nullptr,
                                        (uint32_t*)nullptr, MaxU32(), (int)n, s);
  if (e != hipSuccess) return e;
  const uint64_t o_keys = 0;
  const uint64_t o_rep = o_keys + up(n * 8);
  const uint64_t o_idx = o_rep + up(n * 4);
  const uint64_t o_skeys = o_idx + up(n * 4);
  const uint64_t o_sidx = o_skeys + up(n * 8);
  const uint64_t o_head = o_sidx + up(n * 4);
  const uint64_t o_start = o_head + up(n * 4);
  const uint64_t o_tmp = o_start + up(n * 4);
  const uint64_t total = o_tmp + up(sort_bytes > scan_bytes ? sort_bytes : scan_bytes);
  e = hipMallocAsync(&d.block, total, s);
  if (e != hipSuccess) return e;
  uint8_t* b = (uint8_t*)d.block;
  d.keys = (uint64_t*)(b + o_keys);
  d.rep = (uint32_t*)(b + o_rep);
  uint32_t* idx = (uint32_t*)(b + o_idx);
  uint64_t* skeys = (uint64_t*)(b + o_skeys);
  uint32_t* sidx = (uint32_t*)(b + o_sidx);
  uint32_t* head = (uint32_t*)(b + o_head);
  uint32_t* start = (uint32_t*)(b + o_start);
  void* tmp = b + o_tmp;
  const dim3 grid((unsigned)((n + 255) / 256)), block(256);
  hipLaunchKernelGGL(dedup_init_kernel, grid, block, 0, s, keys, d.keys, idx, n);
  e = hipcub::DeviceRadixSort::SortPairs(tmp, sort_bytes, (const uint64_t*)d.keys, skeys,
                                         (const uint32_t*)idx, sidx, (int)n, 0, 64, s);
  if (e == hipSuccess) {
    hipLaunchKernelGGL(dedup_heads_kernel, grid, block, 0, s, (const uint64_t*)skeys, head, n);
    e = hipcub::DeviceScan::InclusiveScan(tmp, scan_bytes, (const uint32_t*)head, start, MaxU32(),
                                          (int)n, s);
  }
  if (e == hipSuccess) {
    hipLaunchKernelGGL(dedup_mark_kernel, grid, block, 0, s, (const uint32_t*)sidx,
                       (const uint32_t*)start, n, v.empty_key, d.keys, d.rep);
    e = hipGetLastError();
  }
  if (e != hipSuccess) dedup_free(d);
  return e;
}

}  // namespace hkv
#endif
