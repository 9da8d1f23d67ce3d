/*
 * Device helpers shared by the table kernels: addressing, digest matching on
 * packed bytes, 8-lane tile collectives inside a 64-lane wavefront, coherent
 * loads/stores for words that other wavefronts change while a kernel runs.
 * gfx950 only.
 */
#ifndef HKV_COMMON_HPP_
#define HKV_COMMON_HPP_

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "hkv_device.hpp"

namespace hkv {

using View = hkv_table_view;

constexpr uint64_t kMaxScore = UINT64_C(0xFFFFFFFFFFFFFFFF);
constexpr uint64_t kIgnoredEpoch = UINT64_C(0xFFFFFFFFFFFFFFFF);
constexpr uint64_t kEpochMask = UINT64_C(0xFFFFFFFF00000000);
constexpr uint64_t kLow32 = UINT64_C(0xFFFFFFFF);

/* A probe tile is 8 lanes: 8 x 16 bytes cover the 128-byte digest line of a
 * bucket in one fully coalesced load, and a 64-lane wavefront holds 8 tiles. */
constexpr int kTile = 8;
constexpr int kTilesPerWave = kWave / kTile;

/* Everything the probe needs to know about one key of the batch; staged in
 * LDS by the lane that owns the key, read back by the tile that probes it. */
struct KeyMeta {
  uint64_t key;
  uint32_t bkt;
  uint32_t info; /* digest | valid << 8 | start << 16 */
};

/* Bucket, start slot and digest of a key.  get_key_position /
 * get_start_position (kernel_utils.cuh:626-643): global index = hash modulo
 * capacity; digest = hash bits 32..39 (kernel_utils.cuh:84-96).
 *
 * One deliberate difference in the stored byte: a live key whose digest would
 * equal the EMPTY marker stores that value with bit 0 flipped.  The digest
 * array is internal (no API call returns it), lookups apply the same mapping,
 * and an EMPTY-looking byte then always means a slot that was free when the
 * line was read, so a full bucket never costs CAS attempts on live slots. */
__device__ __forceinline__ void locate(const View& v, uint64_t key,
                                       uint32_t& bkt, uint32_t& start,
                                       uint32_t& digest) {
  const uint64_t h = fmix64(key);
  digest = (uint32_t)(h >> 32) & 0xFFu;
  if (digest == v.empty_digest) digest ^= 1u;
  uint64_t g;
  if (v.pow2_buckets)
    g = h & (v.capacity - 1);
  else
    g = h % v.capacity;
  bkt = (uint32_t)(g >> 7);
  start = (uint32_t)(g & 127u) & ~3u;
}

/* 0x80 in every byte of x that is zero, exactly (no borrow artefacts). */
__device__ __forceinline__ uint32_t zero_bytes(uint32_t x) {
  const uint32_t t = (x & 0x7F7F7F7Fu) + 0x7F7F7F7Fu;
  return ~(t | x | 0x7F7F7F7Fu);
}

/*
 * 16-bit match mask of the 16 digest bytes held by a lane against a byte
 * replicated into `pat4`.  Bit (8*b + w) is set when byte b of word w matches
 * ("bw order"); bw_to_pos() turns a bit index back into a byte position.
 */
__device__ __forceinline__ uint32_t match16(const uint4& d, uint32_t pat4) {
  return (zero_bytes(d.x ^ pat4) >> 7) | (zero_bytes(d.y ^ pat4) >> 6) |
         (zero_bytes(d.z ^ pat4) >> 5) | (zero_bytes(d.w ^ pat4) >> 4);
}
__device__ __forceinline__ uint32_t bw_to_pos(uint32_t bit) {
  return ((bit & 7u) << 2) | (bit >> 3);
}

/* ---- 8-lane tile collectives -------------------------------------------- */

template <class T>
__device__ __forceinline__ T tile_bcast(T x, int tile, int j) {
  return __shfl(x, tile * kTile + j);
}
/* 8-bit mask of the lanes of this tile for which pred holds.  Every lane of
 * the tile must be active. */
__device__ __forceinline__ uint32_t tile_ballot(bool pred, int tile) {
  return (uint32_t)(__ballot(pred) >> (tile * kTile)) & 0xFFu;
}

/* ---- coherent access to words other wavefronts may be changing ----------- */

__device__ __forceinline__ uint64_t ld_u64(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u64(uint64_t* p, uint64_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u8(uint8_t* p, uint8_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
/* Slot lock: CAS(expected -> LOCKED) with acquire, as the reference's
 * compare_exchange_strong(…, acquire, relaxed) on the key word
 * (upsert.cuh:104-110). */
__device__ __forceinline__ bool cas_acquire(uint64_t* p, uint64_t expected,
                                            uint64_t desired) {
  return __hip_atomic_compare_exchange_strong(
      p, &expected, desired, __ATOMIC_ACQUIRE, __ATOMIC_RELAXED,
      __HIP_MEMORY_SCOPE_AGENT);
}
/* Slot unlock: release store of the key word (upsert.cuh:228-232). */
__device__ __forceinline__ void st_release(uint64_t* p, uint64_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
}

/* ---- clock ------------------------------------------------------------------ */

struct Clock {
  uint64_t base;        /* deterministic mode: now(i) = base + (i << 20) */
  uint32_t mode;        /* 0 hardware, 1 deterministic */
  uint32_t ns_per_tick; /* hardware mode: constant-rate counter -> ns */
};

/* device_nano (utils.cuh:75-80) */
__device__ __forceinline__ uint64_t now_ns(const Clock& c, uint64_t i) {
  if (c.mode == 1) return c.base + (i << 20);
  return (uint64_t)wall_clock64() * c.ns_per_tick;
}

/* ---- row copies by an 8-lane tile ------------------------------------------ */

template <int VEC>
struct VecType;
template <>
struct VecType<16> {
  using type = uint4;
};
template <>
struct VecType<8> {
  using type = uint2;
};
template <>
struct VecType<4> {
  using type = uint32_t;
};
template <>
struct VecType<2> {
  using type = uint16_t;
};
template <>
struct VecType<1> {
  using type = uint8_t;
};

template <int VEC>
__device__ __forceinline__ void tile_copy(uint8_t* __restrict__ dst,
                                          const uint8_t* __restrict__ src,
                                          uint32_t bytes, int j) {
  using T = typename VecType<VEC>::type;
  const uint32_t units = bytes / VEC;
  T* d = reinterpret_cast<T*>(dst);
  const T* s = reinterpret_cast<const T*>(src);
  uint32_t u = j;
  /* two units in flight per lane */
  for (; u + kTile < units; u += 2 * kTile) {
    T a = s[u];
    T b = s[u + kTile];
    d[u] = a;
    d[u + kTile] = b;
  }
  if (u < units) d[u] = s[u];
}

}  // namespace hkv
#endif
