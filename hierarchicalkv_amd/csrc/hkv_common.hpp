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

/* ---- dual-bucket mode (TableMode::kMemory) ---------------------------------- */

struct DualLoc {
  uint32_t bkt[2];
  uint32_t start[2];
  uint32_t digest;
};

/* get_dual_bucket_indices (dual_bucket_utils.cuh:36-50), the start positions of
 * dual_bucket_upsert.cuh:86-101 (word % capacity, then % 128, rounded down to
 * 4: the capacity is a multiple of 128, so word % 128), digest = hash >> 56.
 * The stored digest byte of a live key never equals the EMPTY marker, as in
 * single-bucket mode (see locate()).  The host side guarantees
 * buckets_num < 2^32. */
__device__ __forceinline__ DualLoc locate_dual(const View& v, uint64_t key) {
  const uint64_t h = fmix64(key);
  const uint32_t lo = (uint32_t)h, hi = (uint32_t)(h >> 32);
  const uint32_t nb = (uint32_t)v.buckets_num;
  DualLoc d;
  if (v.pow2_buckets) {
    d.bkt[0] = lo & (nb - 1);
    d.bkt[1] = hi & (nb - 1);
  } else {
    d.bkt[0] = lo % nb;
    d.bkt[1] = hi % nb;
  }
  if (d.bkt[1] == d.bkt[0]) d.bkt[1] = d.bkt[1] + 1 == nb ? 0 : d.bkt[1] + 1;
  d.start[0] = (lo & 127u) & ~3u;
  d.start[1] = (hi & 127u) & ~3u;
  d.digest = (uint32_t)(h >> 56);
  if (d.digest == v.empty_digest) d.digest ^= 1u;
  return d;
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
/* The same match with bit p set for byte position p (0..15): the four byte
 * flags of a word are gathered into a nibble by one multiply. */
__device__ __forceinline__ uint32_t match16_natural(const uint4& d, uint32_t pat4) {
  const uint32_t n0 = ((zero_bytes(d.x ^ pat4) >> 7) * 0x01020408u) >> 24;
  const uint32_t n1 = ((zero_bytes(d.y ^ pat4) >> 7) * 0x01020408u) >> 24;
  const uint32_t n2 = ((zero_bytes(d.z ^ pat4) >> 7) * 0x01020408u) >> 24;
  const uint32_t n3 = ((zero_bytes(d.w ^ pat4) >> 7) * 0x01020408u) >> 24;
  return n0 | (n1 << 4) | (n2 << 8) | (n3 << 12);
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

/* Value of lane (lane ^ OFF) of the same 8-lane tile, OFF = 1, 2 or 4, by data-parallel moves
 * inside the vector unit: no trip through the LDS permute network as with __shfl_xor, whose
 * latency adds up in the reductions that sit in dependent chains.  Every lane of the tile must
 * be active.  lane ^ 4 is the mirror image of the 8 lanes followed by the mirror image of each
 * quad. */
template <int OFF>
__device__ __forceinline__ uint32_t tile_xor(uint32_t x) {
  static_assert(OFF == 1 || OFF == 2 || OFF == 4, "inside a tile");
  if constexpr (OFF == 1) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, true); /* quad_perm [1,0,3,2] */
  if constexpr (OFF == 2) return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, true); /* quad_perm [2,3,0,1] */
  const int h = __builtin_amdgcn_update_dpp(0, (int)x, 0x141, 0xF, 0xF, true); /* row_half_mirror */
  return (uint32_t)__builtin_amdgcn_update_dpp(0, h, 0x1B, 0xF, 0xF, true);     /* quad_perm [3,2,1,0] */
}
template <int OFF>
__device__ __forceinline__ uint64_t tile_xor(uint64_t x) {
  return tile_xor<OFF>((uint32_t)x) | ((uint64_t)tile_xor<OFF>((uint32_t)(x >> 32)) << 32);
}
/* Minimum of a 64-bit value over the tile, and of (value, position) pairs ordered by value, then
 * position; selects, no branches. */
__device__ __forceinline__ uint64_t tile_min(uint64_t m) {
  uint64_t o = tile_xor<1>(m);
  m = o < m ? o : m;
  o = tile_xor<2>(m);
  m = o < m ? o : m;
  o = tile_xor<4>(m);
  return o < m ? o : m;
}
template <int OFF>
__device__ __forceinline__ void tile_min_pair_step(uint64_t& m, uint32_t& pos) {
  const uint64_t om = tile_xor<OFF>(m);
  const uint32_t op = tile_xor<OFF>(pos);
  const bool take = om < m || (om == m && op < pos);
  m = take ? om : m;
  pos = take ? op : pos;
}
__device__ __forceinline__ void tile_min_pair(uint64_t& m, uint32_t& pos) {
  tile_min_pair_step<1>(m, pos);
  tile_min_pair_step<2>(m, pos);
  tile_min_pair_step<4>(m, pos);
}

/* ---- coherent access to words other wavefronts may be changing -----------
 *
 * An MI355X has one L2 per XCD (8 of them); ordinary cached loads and stores
 * are only coherent inside one XCD until a kernel ends.  Acquire / release at
 * agent scope would make the compiler write back and invalidate the whole L2
 * around every slot lock, which costs far more than the lock protects.  So the
 * protocol is built from agent-scope *relaxed* accesses instead: such loads
 * and stores carry the sc1 bit, i.e. stores write through to memory and loads
 * do not trust a line another XCD may have changed.  Everything a second
 * wavefront may read or overwrite while this kernel runs (key words, digests,
 * scores, and value rows of the table) goes through these helpers; the unlock
 * waits for the wavefront's outstanding stores first (wait_stores). */

__device__ __forceinline__ uint64_t ld_u64(const uint64_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint32_t ld_u32(const uint32_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ uint8_t ld_u8(const uint8_t* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u64(uint64_t* p, uint64_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u32(uint32_t* p, uint32_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st_u8(uint8_t* p, uint8_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
/* 16-byte agent-coherent load at byte `offset` of an array of `bytes` bytes (below 4 GiB),
 * as one instruction.  The compiler offers 128-bit agent-scope loads only through a buffer
 * resource; the array's base and size are the same for the whole wavefront, the offset is
 * per lane.  Offsets past the end read zero. */
__device__ __forceinline__ uint4 ld_u128_at(const void* base, uint64_t bytes, uint64_t offset) {
  const __amdgpu_buffer_rsrc_t rs =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (uint32_t)bytes, 0x00020000);
  const u32x4_t x = __builtin_amdgcn_raw_buffer_load_b128(rs, (uint32_t)offset, 0, 16 /* sc1 */);
  return make_uint4(x.x, x.y, x.z, x.w);
}
/* 16-byte write-through store, marked non-temporal: what is written this way (value
 * rows, a whole digest line) is not read again soon, and keeping it out of the caches
 * leaves them to the digest and key lines the next call probes (measured: the next find
 * runs 8 % faster, the upsert itself 4 %).  The compiler has no 128-bit agent-scope store,
 * and two 8-byte ones per lane interleave inside a 128-byte line, which the
 * memory side then writes as two half-filled lines each.  The instruction is
 * issued from inline assembly: the wavefront's store counter still covers it
 * (wait_stores).  On gfx940 and later a store of more than 64 bits needs two wait states
 * before a VALU instruction may overwrite its data registers; the compiler's hazard
 * recognizer does not look inside inline assembly, so the s_nop 1 (two wait states)
 * provides them whatever gets scheduled next. */
__device__ __forceinline__ void st_u128(void* p, const uint4& x) {
  u32x4_t d = {x.x, x.y, x.z, x.w};
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(d) : "memory");
}
/* Slot lock: CAS(expected -> LOCKED) on the key word (the reference's
 * compare_exchange_strong, upsert.cuh:104-110).  On failure `expected` holds
 * the word that was found. */
__device__ __forceinline__ bool cas_lock(uint64_t* p, uint64_t& expected,
                                         uint64_t desired) {
  return __hip_atomic_compare_exchange_strong(p, &expected, desired,
                                              __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                              __HIP_MEMORY_SCOPE_AGENT);
}
/* Slot lock without knowing what the slot holds: the key word becomes LOCKED and its
 * previous content comes back. */
__device__ __forceinline__ uint64_t swap_lock(uint64_t* p, uint64_t locked) {
  return __hip_atomic_exchange(p, locked, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
/* Every store this wavefront has issued is complete (written through) and the
 * compiler moves no memory access across this point. */
__device__ __forceinline__ void wait_stores() {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}
/* Slot unlock: the key word becomes visible after everything written under
 * the lock (the reference's release store, upsert.cuh:228-232).  The caller
 * has executed wait_stores() with all lanes of the tile active. */
__device__ __forceinline__ void st_unlock(uint64_t* p, uint64_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

/* The table's count of slots that lock_keys and the pointer overload with locked_key_ptrs have left
 * LOCKED is kept in kLockedShards words, each in a 128-byte line of its own, and a workgroup
 * adds to the word of its index: updates of one word are served one at a time, about 13 ns
 * each, and one word for the 16 384 wavefronts of 2^20 keys was 0.21 ms of a 0.24 ms lock_keys. */
constexpr unsigned kLockedShards = 64;
constexpr unsigned kLockedStride = 16; /* words */
__device__ __forceinline__ unsigned long long* locked_shard(unsigned long long* count) {
  return count + (blockIdx.x & (kLockedShards - 1)) * kLockedStride;
}

/* ---- clock ------------------------------------------------------------------ */

struct Clock {
  uint64_t base;        /* deterministic mode: now(i) = base + (i << 20) */
  uint64_t offset;      /* hardware mode: Unix-epoch ns at tick 0 of the device counter */
  uint32_t mode;        /* 0 hardware, 1 deterministic */
  uint32_t ns_per_tick; /* hardware mode: constant-rate counter -> ns */
};

/* device_nano (utils.cuh:75-80): the reference reads %globaltimer, nanoseconds since the Unix
 * epoch.  The constant-rate counter of the device restarts with the device, so the table keeps
 * the epoch time of its tick 0 (sampled against the host's CLOCK_REALTIME when the table is
 * created): scores stay comparable with host time, across processes and after load(). */
__device__ __forceinline__ uint64_t now_ns(const Clock& c, uint64_t i) {
  if (c.mode == 1) return c.base + (i << 20);
  return c.offset + (uint64_t)wall_clock64() * c.ns_per_tick;
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

/* Row copy by the 8 lanes of a tile, VEC bytes per lane and trip (16, 4 or 1).
 * DST_TABLE / SRC_TABLE say which side is a value row of the table and must be
 * accessed coherently (8-, 4- or 1-byte agent-scope accesses); the caller's
 * buffers are accessed with plain VEC-wide loads and stores. */
template <int VEC, bool DST_TABLE, bool SRC_TABLE>
__device__ __forceinline__ void tile_copy(uint8_t* __restrict__ dst,
                                          const uint8_t* __restrict__ src,
                                          uint32_t bytes, int j) {
  const uint32_t units = bytes / VEC;
  if (VEC == 16) {
    for (uint32_t u = j; u < units; u += 2 * kTile) {
      const uint32_t u2 = u + kTile;
      const bool two = u2 < units;
      uint64_t a0, a1, b0 = 0, b1 = 0;
      if (SRC_TABLE) {
        const uint64_t* s = reinterpret_cast<const uint64_t*>(src);
        a0 = ld_u64(s + 2 * u);
        a1 = ld_u64(s + 2 * u + 1);
        if (two) {
          b0 = ld_u64(s + 2 * u2);
          b1 = ld_u64(s + 2 * u2 + 1);
        }
      } else {
        const uint4* s = reinterpret_cast<const uint4*>(src);
        const uint4 a = s[u];
        a0 = a.x | ((uint64_t)a.y << 32);
        a1 = a.z | ((uint64_t)a.w << 32);
        if (two) {
          const uint4 b = s[u2];
          b0 = b.x | ((uint64_t)b.y << 32);
          b1 = b.z | ((uint64_t)b.w << 32);
        }
      }
      if (DST_TABLE) {
        uint64_t* d = reinterpret_cast<uint64_t*>(dst);
        st_u64(d + 2 * u, a0);
        st_u64(d + 2 * u + 1, a1);
        if (two) {
          st_u64(d + 2 * u2, b0);
          st_u64(d + 2 * u2 + 1, b1);
        }
      } else {
        uint4* d = reinterpret_cast<uint4*>(dst);
        d[u] = make_uint4((uint32_t)a0, (uint32_t)(a0 >> 32), (uint32_t)a1, (uint32_t)(a1 >> 32));
        if (two)
          d[u2] = make_uint4((uint32_t)b0, (uint32_t)(b0 >> 32), (uint32_t)b1, (uint32_t)(b1 >> 32));
      }
    }
  } else if (VEC == 4) {
    const uint32_t* s = reinterpret_cast<const uint32_t*>(src);
    uint32_t* d = reinterpret_cast<uint32_t*>(dst);
    for (uint32_t u = j; u < units; u += kTile) {
      const uint32_t x = SRC_TABLE ? ld_u32(s + u) : s[u];
      if (DST_TABLE)
        st_u32(d + u, x);
      else
        d[u] = x;
    }
  } else {
    for (uint32_t u = j; u < units; u += kTile) {
      const uint8_t x = SRC_TABLE ? ld_u8(src + u) : src[u];
      if (DST_TABLE)
        st_u8(dst + u, x);
      else
        dst[u] = x;
    }
  }
}

}  // namespace hkv
#endif
