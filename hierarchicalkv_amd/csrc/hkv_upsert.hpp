/*
 * The upsert family: insert_or_assign, insert_and_evict, find_or_insert
 * (values and pointers), accum_or_assign, and the assign family.  One kernel
 * template for every load factor; one 64-lane wavefront per workgroup,
 * 64 keys per wavefront.
 *
 * Replaces tlp_v1/tlp_v2/pipeline_upsert_kernel_with_io (upsert.cuh:27-986),
 * the *_upsert_and_evict_kernel_unique kernels (upsert_and_evict.cuh:27-1099),
 * the find_or_insert kernels (find_or_insert.cuh:27-1050), the pointer kernel
 * (find_ptr_or_insert.cuh:27-246), accum_or_assign_kernel_with_io
 * (accum_or_assign.cuh:83-174) and the update kernels (update.cuh,
 * update_score.cuh, update_values.cuh).  Per-key semantics follow
 * upsert.cuh:52-233.
 *
 * Division of labour inside a wavefront
 *   control  lane L owns key L: it decides what to lock, issues the 64-bit CAS
 *            on the key word, writes digest / score, and unlocks.  All 64 keys
 *            take each of these steps in one instruction, so a wavefront pays
 *            one memory round trip per step, not one per key.
 *   bulk     tile t (lanes 8t..8t+7) serves the keys 8t..8t+7 of its own
 *            lanes: the digest probe (hkv_lookup.hpp), the min-score scan of a
 *            full bucket (16 scores per lane, 8 coalesced 128-byte lines per
 *            tile, reduce inside the lane and then over the tile) and the
 *            value-row copies, issued for several keys before the first result
 *            is awaited.  How much is in flight per wavefront is weighed
 *            against registers: at 118 registers four wavefronts share a SIMD,
 *            and that is worth more here than deeper batches per wavefront.
 *
 * Lock discipline on a SIMD machine: every lock taken in a trip of the retry
 * loop is released at the end of the same trip, and the loop's exit test is a
 * wavefront-wide ballot.  A lane that found a slot LOCKED by another lane of
 * its wavefront therefore always finds it released on its next trip.
 */
#ifndef HKV_UPSERT_HPP_
#define HKV_UPSERT_HPP_

#include "hkv_lookup.hpp"

namespace hkv {

enum UpsertOp {
  kOpInsertOrAssign = 0,
  kOpInsertAndEvict = 1,
  kOpFindOrInsert = 2,
  kOpAccumOrAssign = 3,
  kOpFindOrInsertPtr = 4,
};

struct UpsertArgs {
  const uint64_t* keys;
  const uint8_t* values_in;  /* insert_or_assign, insert_and_evict, accum */
  uint8_t* values_io;        /* find_or_insert */
  const uint64_t* scores;    /* may be null (LRU, EpochLRU) */
  const uint8_t* accum_flags;
  uint64_t* evicted_keys;
  uint8_t* evicted_values;
  uint64_t* evicted_scores;  /* may be null */
  unsigned long long* evicted_counter;
  void** out_ptrs;           /* find_or_insert pointer overload */
  uint64_t** locked_key_ptrs; /* same overload: when given, the slots stay LOCKED and their key
                                 addresses go here (find_ptr_or_insert.cuh:232-242) */
  uint8_t* founds;
  unsigned long long* locked_count;   /* with locked_key_ptrs: the table's count of slots left LOCKED */
  uint64_t* held_scores;              /* the upserts of hybrid mode (the other overloads with locked_key_ptrs):
                                         the score of every slot that is left LOCKED; the slot itself
                                         shows kMaxScore until the launch that opens it */
  uint64_t n;
  uint64_t epoch;
  Clock clock;
  int32_t value_kind;
  int32_t strategy; /* hkv_evict_strategy; uniform, so a scalar branch */
  int32_t refuse_equal; /* refuse when score <= min instead of < (hybrid and
                           pointer kernels, upsert.cuh:1524, find_or_insert.cuh:1593) */
  /* score bounds (BOUNDS kernels): no bound is set above `bound_cap`, or above *bound_cap_in
   * when that is given; the kernel leaves a clock reading in *bound_cap_out for the next call */
  uint64_t bound_cap;
  const unsigned long long* bound_cap_in;
  unsigned long long* bound_cap_out;
  /* strategies whose scores come from the caller (Customized, LFU, EpochLFU): a device word that
   * no bound of the table is above.  A key that writes a score below it lowers the bound of
   * its line itself.  Null where scores only grow (LRU, EpochLRU). */
  unsigned long long* bound_ceil;
};

/* ScoreFunctor<Strategy>::desired_when_missed, kernel_utils.cuh:275-279,
 * 332-336, 403-411, 464-471, 567-571 */
__device__ __forceinline__ uint64_t desired_when_missed(const UpsertArgs& a,
                                                        uint64_t in_score,
                                                        uint64_t i) {
  const int STRATEGY = a.strategy;
  if (STRATEGY == HKV_LRU) return now_ns(a.clock, i);
  if (STRATEGY == HKV_LFU) return kMaxScore;
  if (STRATEGY == HKV_EPOCH_LRU) {
    if (a.epoch == kIgnoredEpoch && a.scores) return in_score;
    return (a.epoch << 32) | ((now_ns(a.clock, i) >> 20) & kLow32);
  }
  if (STRATEGY == HKV_EPOCH_LFU) {
    if (a.epoch == kIgnoredEpoch) return in_score;
    return (a.epoch << 32) | (in_score & kLow32);
  }
  return in_score;
}

/* ScoreFunctor<Strategy>::update_with_digest, kernel_utils.cuh:291-302,
 * 353-371, 422-434, 490-517, 581-593: digest and score of an accepted key.
 * The slot is locked by the caller. */
__device__ __forceinline__ uint64_t write_meta(const View& v, const UpsertArgs& a,
                                               uint64_t slot, uint32_t digest,
                                               uint64_t desired, uint64_t in_score,
                                               uint64_t i, bool new_insert, bool hold = false) {
  const int STRATEGY = a.strategy;
  uint64_t s = desired;
  if (STRATEGY == HKV_LRU) {
    s = now_ns(a.clock, i);
  } else if (STRATEGY == HKV_LFU) {
    if (!a.scores) return kMaxScore;
    s = new_insert ? in_score : in_score + ld_u64(v.scores + slot);
  } else if (STRATEGY == HKV_EPOCH_LFU) {
    if (!new_insert) {
      s = ld_u64(v.scores + slot) & kLow32;
      if (kLow32 - s > (desired & kLow32))
        s += desired;
      else
        s = (desired & kEpochMask) | kLow32;
    }
  }
  /* a hit keeps its digest: the byte is only written when the slot changes
   * owner (the reference rewrites the same value, kernel_utils.cuh:296-300) */
  if (new_insert) st_u8(v.digests + slot, (uint8_t)digest);
  /* `hold`: the slot stays LOCKED to the end of the launch and must not look like a victim to
   * the searches that read scores only; the caller keeps `s` for the launch that opens it */
  st_u64(v.scores + slot, hold ? kMaxScore : s);
  return s; /* what the slot holds in the end (kMaxScore above: nothing was written) */
}

/* wrapping adds of the 8- and 16-bit lanes of a word (signed and unsigned alike) */
__device__ __forceinline__ uint32_t add_lanes8(uint32_t x, uint32_t y) {
  return ((x & 0x7F7F7F7Fu) + (y & 0x7F7F7F7Fu)) ^ ((x ^ y) & 0x80808080u);
}
__device__ __forceinline__ uint32_t add_lanes16(uint32_t x, uint32_t y) {
  return ((x & 0x7FFF7FFFu) + (y & 0x7FFF7FFFu)) ^ ((x ^ y) & 0x80008000u);
}
/* x + y on one unit of a row, element type by `kind` (accum_or_assign_vector,
 * accum_or_assign.cuh:24-35); one IEEE add per element. */
__device__ __forceinline__ uint4 add_unit(uint4 x, uint4 y, int kind) {
  if (kind == HKV_VALUE_F32) {
    x.x = __float_as_uint(__uint_as_float(x.x) + __uint_as_float(y.x));
    x.y = __float_as_uint(__uint_as_float(x.y) + __uint_as_float(y.y));
    x.z = __float_as_uint(__uint_as_float(x.z) + __uint_as_float(y.z));
    x.w = __float_as_uint(__uint_as_float(x.w) + __uint_as_float(y.w));
  } else if (kind == HKV_VALUE_I8) {
    x = make_uint4(add_lanes8(x.x, y.x), add_lanes8(x.y, y.y), add_lanes8(x.z, y.z), add_lanes8(x.w, y.w));
  } else if (kind == HKV_VALUE_I16) {
    x = make_uint4(add_lanes16(x.x, y.x), add_lanes16(x.y, y.y), add_lanes16(x.z, y.z), add_lanes16(x.w, y.w));
  } else if (kind == HKV_VALUE_I32) {
    x.x += y.x;
    x.y += y.y;
    x.z += y.z;
    x.w += y.w;
  } else {
    uint64_t a0 = x.x | ((uint64_t)x.y << 32), a1 = x.z | ((uint64_t)x.w << 32);
    const uint64_t b0 = y.x | ((uint64_t)y.y << 32), b1 = y.z | ((uint64_t)y.w << 32);
    if (kind == HKV_VALUE_F64) {
      a0 = (uint64_t)__double_as_longlong(__longlong_as_double((long long)a0) +
                                          __longlong_as_double((long long)b0));
      a1 = (uint64_t)__double_as_longlong(__longlong_as_double((long long)a1) +
                                          __longlong_as_double((long long)b1));
    } else {
      a0 += b0;
      a1 += b1;
    }
    x = make_uint4((uint32_t)a0, (uint32_t)(a0 >> 32), (uint32_t)a1, (uint32_t)(a1 >> 32));
  }
  return x;
}
/* The host side picks a unit that is at least one element wide (accum_unit in hkv_table.hip). */
__device__ __forceinline__ uint32_t add_unit(uint32_t x, uint32_t y, int kind) {
  if (kind == HKV_VALUE_F32) return __float_as_uint(__uint_as_float(x) + __uint_as_float(y));
  if (kind == HKV_VALUE_I8) return add_lanes8(x, y);
  if (kind == HKV_VALUE_I16) return add_lanes16(x, y);
  return x + y; /* i32 */
}
__device__ __forceinline__ uint2 add_unit(uint2 x, uint2 y, int kind) {
  if (kind == HKV_VALUE_F64 || kind == HKV_VALUE_I64) {
    uint64_t a = x.x | ((uint64_t)x.y << 32);
    const uint64_t b = y.x | ((uint64_t)y.y << 32);
    if (kind == HKV_VALUE_F64)
      a = (uint64_t)__double_as_longlong(__longlong_as_double((long long)a) +
                                         __longlong_as_double((long long)b));
    else
      a += b;
    return make_uint2((uint32_t)a, (uint32_t)(a >> 32));
  }
  return make_uint2(add_unit(x.x, y.x, kind), add_unit(x.y, y.y, kind));
}
__device__ __forceinline__ uint16_t add_unit(uint16_t x, uint16_t y, int kind) {
  if (kind == HKV_VALUE_I8) return (uint16_t)add_lanes8(x, y);
  return (uint16_t)(x + y); /* i16 */
}
__device__ __forceinline__ uint8_t add_unit(uint8_t x, uint8_t y, int) {
  return (uint8_t)(x + y); /* i8 */
}

/* One VEC-byte unit of a row.  Table rows are read and written coherently
 * (agent-scope accesses: 2 x 8 bytes per 16-byte unit on the load side, one
 * 16-byte write-through store on the store side), caller buffers plainly. */
template <int VEC, bool TABLE>
__device__ __forceinline__ typename VecType<VEC>::type ld_unit(const uint8_t* row, uint32_t u) {
  using T = typename VecType<VEC>::type;
  if constexpr (!TABLE) {
    if constexpr (VEC == 16) {
      /* a caller's row is read once: streaming load, so that it does not push table
       * lines out of the caches */
      const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(row) + u);
      return make_uint4(t.x, t.y, t.z, t.w);
    } else {
      return reinterpret_cast<const T*>(row)[u];
    }
  } else if constexpr (VEC == 16) {
    const uint64_t* p = reinterpret_cast<const uint64_t*>(row) + 2 * u;
    const uint64_t lo = ld_u64(p), hi = ld_u64(p + 1);
    return make_uint4((uint32_t)lo, (uint32_t)(lo >> 32), (uint32_t)hi, (uint32_t)(hi >> 32));
  } else if constexpr (VEC == 8) {
    const uint64_t x = ld_u64(reinterpret_cast<const uint64_t*>(row) + u);
    return make_uint2((uint32_t)x, (uint32_t)(x >> 32));
  } else if constexpr (VEC == 4) {
    return ld_u32(reinterpret_cast<const uint32_t*>(row) + u);
  } else if constexpr (VEC == 2) {
    return __hip_atomic_load(reinterpret_cast<const uint16_t*>(row) + u, __ATOMIC_RELAXED,
                             __HIP_MEMORY_SCOPE_AGENT);
  } else {
    return ld_u8(row + u);
  }
}
template <int VEC, bool TABLE>
__device__ __forceinline__ void st_unit(uint8_t* row, uint32_t u, typename VecType<VEC>::type x) {
  using T = typename VecType<VEC>::type;
  if constexpr (!TABLE) {
    if constexpr (VEC == 16) {
      /* written once, not read again by this kernel: streaming store */
      const u32x4_t t = {x.x, x.y, x.z, x.w};
      __builtin_nontemporal_store(t, reinterpret_cast<u32x4_t*>(row) + u);
    } else {
      reinterpret_cast<T*>(row)[u] = x;
    }
  } else if constexpr (VEC == 16) {
    st_u128(row + 16 * (size_t)u, x);
  } else if constexpr (VEC == 8) {
    st_u64(reinterpret_cast<uint64_t*>(row) + u, x.x | ((uint64_t)x.y << 32));
  } else if constexpr (VEC == 4) {
    st_u32(reinterpret_cast<uint32_t*>(row) + u, x);
  } else if constexpr (VEC == 2) {
    __hip_atomic_store(reinterpret_cast<uint16_t*>(row) + u, x, __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
  } else {
    st_u8(row + u, x);
  }
}

enum : int {
  kStNone = 0, /* no lock taken (yet) */
  kStDuplicate = 1,
  kStEmpty = 2,
  kStReclaimed = 3,
  kStEvict = 4,
  kStRefused = 5,
  kStAbsent = 6, /* assign family: key not in the table */
};

/* what the bulk phase has to move for a key in this trip */
enum : int {
  kMoveNone = 0,
  kMoveInToTable = 1,  /* caller's row -> table row */
  kMoveTableToIo = 2,  /* table row -> caller's row (find_or_insert hit) */
  kMoveAccum = 3,      /* table row += caller's row */
};

/* first set bit of a 128-bit mask at or after bit `s` (wrapping); the mask is
 * not zero */
__device__ __forceinline__ uint32_t first_from(uint64_t lo, uint64_t hi, uint32_t s) {
  if (s & 64) {
    const uint64_t t = lo;
    lo = hi;
    hi = t;
  }
  const uint32_t sh = s & 63;
  uint64_t rlo = lo, rhi = hi;
  if (sh) {
    rlo = (lo >> sh) | (hi << (64 - sh));
    rhi = (hi >> sh) | (lo << (64 - sh));
  }
  const uint32_t idx = rlo ? (uint32_t)__ffsll((unsigned long long)rlo) - 1
                           : 64 + (uint32_t)__ffsll((unsigned long long)rhi) - 1;
  return (idx + s) & 127u;
}

/*
 * Min-score scan of a bucket by the 8 lanes of a tile: the loads, then the reduction.
 * Lane j holds scores {16 it + 2j, 16 it + 2j + 1 : it = 0..7}: each `it` is
 * one coalesced 128-byte line per tile.  LOCKED_RULE hides slots whose key is
 * LOCKED or EMPTY (find_ptr_or_insert.cuh:170-180).
 */
template <bool LOCKED_RULE>
__device__ __forceinline__ void scan_load(const View& v, uint64_t bslot, int j, uint64_t* sc,
                                          uint64_t* kc) {
  if (v.capacity < (UINT64_C(1) << 29)) {
    /* one 16-byte coherent load per line and lane (ld_u128_at): half the load instructions
     * of the 8-byte form, measured 6 % on a whole insert_or_assign batch */
#pragma unroll
    for (int it = 0; it < kTile; it++) {
      const uint4 x = ld_u128_at(v.scores, v.capacity * 8, (bslot + it * 16 + j * 2) * 8);
      sc[2 * it] = x.x | ((uint64_t)x.y << 32);
      sc[2 * it + 1] = x.z | ((uint64_t)x.w << 32);
    }
    if (LOCKED_RULE) {
#pragma unroll
      for (int it = 0; it < kTile; it++) {
        const uint4 x = ld_u128_at(v.keys, v.capacity * 8, (bslot + it * 16 + j * 2) * 8);
        kc[2 * it] = x.x | ((uint64_t)x.y << 32);
        kc[2 * it + 1] = x.z | ((uint64_t)x.w << 32);
      }
    }
    return;
  }
#pragma unroll
  for (int it = 0; it < kTile; it++) {
    const uint64_t* sp = v.scores + bslot + it * 16 + j * 2;
    sc[2 * it] = ld_u64(sp);
    sc[2 * it + 1] = ld_u64(sp + 1);
  }
  if (LOCKED_RULE) {
#pragma unroll
    for (int it = 0; it < kTile; it++) {
      const uint64_t* kp = v.keys + bslot + it * 16 + j * 2;
      kc[2 * it] = ld_u64(kp);
      kc[2 * it + 1] = ld_u64(kp + 1);
    }
  }
}
/* ties go to the lowest slot, as the reference's sequential scan with a strict
 * '<' (upsert.cuh:166-183) */
template <bool LOCKED_RULE>
__device__ __forceinline__ void scan_reduce(const View& v, const uint64_t* sc, const uint64_t* kc,
                                            int j, uint64_t& best, uint32_t& bpos) {
  best = kMaxScore;
  bpos = 0;
#pragma unroll
  for (int q = 0; q < 2 * kTile; q++) {
    uint64_t s = sc[q];
    if (LOCKED_RULE && (kc[q] == v.locked_key || kc[q] == v.empty_key)) s = kMaxScore;
    const uint32_t p = (q >> 1) * 16 + j * 2 + (q & 1);
    if (s < best) {
      best = s;
      bpos = p;
    }
  }
  tile_min_pair(best, bpos);
}

/* ---- min-score search with per-line lower bounds (LRU) -------------------------------------------
 * v.bounds holds, for every line of 16 scores, a value that is not above any score in the line.
 * Under LRU a score only ever grows (a touched or new key gets the current time), so a bound
 * that was right once stays right without anybody maintaining it, and 0 is always right.  The
 * tile reads the bucket's 8 bounds (64 bytes), then only the score line with the lowest bound:
 * if that line's minimum is not above any other line's bound it is the bucket's minimum, found
 * with 2 line reads instead of 8.  Otherwise the lines whose bound is below the best score so
 * far are opened one by one (and their bounds set to what they hold).  The result is the slot a
 * scan of all 128 scores returns (ties to the lowest slot).
 * "Only grows" holds from call to call, not inside one: keys of one batch get their scores in no
 * particular order.  So no bound is ever set above `cap`, a value no score of the running call
 * is below (the base of the deterministic clock, or a clock reading from before the call). */

/* the two scores of lane j in line g of the bucket at slot `bs` */
__device__ __forceinline__ uint4 line_load(const View& v, uint64_t bs, uint32_t g, int j) {
  const uint64_t at = bs + g * 16 + j * 2;
  if (v.capacity < (UINT64_C(1) << 29)) return ld_u128_at(v.scores, v.capacity * 8, at * 8);
  const uint64_t a = ld_u64(v.scores + at), b = ld_u64(v.scores + at + 1);
  return make_uint4((uint32_t)a, (uint32_t)(a >> 32), (uint32_t)b, (uint32_t)(b >> 32));
}
/* minimum of line g over the tile: score and slot position in the bucket */
__device__ __forceinline__ void line_min(const uint4& x, uint32_t g, int j, uint64_t& m, uint32_t& pos) {
  const uint64_t s0 = x.x | ((uint64_t)x.y << 32), s1 = x.z | ((uint64_t)x.w << 32);
  const uint32_t p0 = g * 16 + j * 2;
  m = s1 < s0 ? s1 : s0;
  pos = s1 < s0 ? p0 + 1 : p0;
  tile_min_pair(m, pos);
}
/* `bd`: this lane's bound (line j); `g`, `x`: the line with the lowest bound and this lane's
 * part of it.  All 8 lanes of the tile call this together.  `nb`: what line bpos / 16 is bounded
 * by once slot bpos has been given a score that is above everything else in it. */
__device__ __forceinline__ void bounded_min(const View& v, uint64_t bs, int tile, int j, uint64_t bd,
                                            uint32_t g, uint4 x, uint64_t cap, uint64_t& best,
                                            uint32_t& bpos, uint64_t& nb) {
  uint64_t* const bounds = v.bounds + (bs >> 4);
  line_min(x, g, j, best, bpos);
  uint32_t opened = 1u << g;
  for (;;) {
    const bool lower = !((opened >> j) & 1u) && (bd < best || (bd == best && (uint32_t)j < (bpos >> 4)));
    const uint32_t cand = tile_ballot(lower, tile);
    if (!cand) break;
    const uint32_t c = (uint32_t)__ffs(cand) - 1;
    opened |= 1u << c;
    const uint4 y = line_load(v, bs, c, j);
    uint64_t m;
    uint32_t pos;
    line_min(y, c, j, m, pos);
    if (m < best || (m == best && pos < bpos)) {
      /* the line that held the best so far is bounded by exactly that */
      if ((uint32_t)j == (bpos >> 4)) st_u64(bounds + j, best < cap ? best : cap);
      best = m;
      bpos = pos;
      x = y;
    } else if ((uint32_t)j == c) {
      st_u64(bounds + c, m < cap ? m : cap);
    }
  }
  /* the smallest score of the chosen line apart from the chosen slot */
  const uint64_t s0 = x.x | ((uint64_t)x.y << 32), s1 = x.z | ((uint64_t)x.w << 32);
  const uint32_t p0 = (bpos & ~15u) + j * 2;
  const uint64_t r0 = p0 == bpos ? kMaxScore : s0, r1 = p0 + 1 == bpos ? kMaxScore : s1;
  nb = tile_min(r1 < r0 ? r1 : r0);
}

/* 16-byte units of value rows a lane holds in registers at a time in the bulk copies.  Fewer
 * means fewer row loads in flight per wavefront but also fewer registers, i.e. more wavefronts
 * per SIMD; measured on insert_or_assign (rows of 256 bytes): 16 units 0.323 ms, 8 units
 * 0.306 ms per 2^20 keys. */
constexpr int kRowUnits = 8;

/*
 * Bulk row traffic of one trip.  Round q of a tile is the key owned by lane q
 * of the tile: `move` says what to do with it, `tab` is its table row, `usr`
 * the caller's row.  All loads of a group of rounds are issued before the
 * first store; a group holds 16 units per lane (64 VGPRs at 16-byte units),
 * i.e. the whole trip for rows up to 256 bytes.
 * UPL = units per lane and row held in registers (1, 2, 4 or 8).
 * Every lane of the wavefront must call this.
 */
template <int VEC, int UPL, bool CAN_READ_TABLE, bool CAN_ACCUM>
__device__ __forceinline__ void bulk_rows(int move, uint8_t* tab, uint8_t* usr,
                                          uint32_t units, int value_kind, int lane) {
  using T = typename VecType<VEC>::type;
  /* accumulating holds two rows per key (the table's and the caller's): half as many keys at a time */
  constexpr int kUnits = CAN_ACCUM ? kRowUnits / 2 : kRowUnits;
  constexpr int kGroup = kUnits / UPL < 1 ? 1 : (kUnits / UPL < kTile ? kUnits / UPL : kTile);
  const int j = lane & (kTile - 1);
  const int lane_base = lane & ~(kTile - 1);
  for (uint32_t u0 = 0; u0 < units; u0 += kTile * UPL) {
#pragma unroll
    for (int g = 0; g < kTile; g += kGroup) {
      T x[kGroup][UPL];
      T y[CAN_ACCUM ? kGroup : 1][CAN_ACCUM ? UPL : 1];
#pragma unroll
      for (int q = 0; q < kGroup; q++) {
        const int src = lane_base + g + q;
        const int mv = __shfl(move, src);
        const uint8_t* tb = reinterpret_cast<const uint8_t*>(__shfl((unsigned long long)tab, src));
        const uint8_t* us = reinterpret_cast<const uint8_t*>(__shfl((unsigned long long)usr, src));
#pragma unroll
        for (int w = 0; w < UPL; w++) {
          const uint32_t u = u0 + j + w * kTile;
          x[q][w] = T{};
          if (u < units) {
            if (mv == kMoveInToTable) x[q][w] = ld_unit<VEC, false>(us, u);
            /* the row of a key that was found was last written before this launch (keys are
             * unique, so no other key of the batch has touched it): an ordinary streaming
             * load, one 16-byte access instead of the two 8-byte coherent ones */
            if (CAN_READ_TABLE && mv == kMoveTableToIo) x[q][w] = ld_unit<VEC, false>(tb, u);
            if (CAN_ACCUM && mv == kMoveAccum) {
              x[q][w] = ld_unit<VEC, false>(tb, u);
              y[q][w] = ld_unit<VEC, false>(us, u);
            }
          }
        }
      }
#pragma unroll
      for (int q = 0; q < kGroup; q++) {
        const int src = lane_base + g + q;
        const int mv = __shfl(move, src);
        uint8_t* tb = reinterpret_cast<uint8_t*>(__shfl((unsigned long long)tab, src));
        uint8_t* us = reinterpret_cast<uint8_t*>(__shfl((unsigned long long)usr, src));
#pragma unroll
        for (int w = 0; w < UPL; w++) {
          const uint32_t u = u0 + j + w * kTile;
          if (u < units) {
            if (mv == kMoveInToTable) st_unit<VEC, true>(tb, u, x[q][w]);
            if (CAN_READ_TABLE && mv == kMoveTableToIo) st_unit<VEC, false>(us, u, x[q][w]);
            if (CAN_ACCUM && mv == kMoveAccum)
              st_unit<VEC, true>(tb, u, add_unit(x[q][w], y[q][w], value_kind));
          }
        }
      }
    }
  }
}

/* Copies towards the evicted-values output: kind 2 = the victim's table row
 * (coherent read), kind 1 = the refused key's input row, 0 = nothing. */
template <int VEC, int UPL>
__device__ __forceinline__ void bulk_evicted(int kind, const uint8_t* src, uint8_t* dst,
                                             uint32_t units, int lane) {
  using T = typename VecType<VEC>::type;
  constexpr int kGroup = kRowUnits / UPL < 1 ? 1 : (kRowUnits / UPL < kTile ? kRowUnits / UPL : kTile);
  const int j = lane & (kTile - 1);
  const int lane_base = lane & ~(kTile - 1);
  for (uint32_t u0 = 0; u0 < units; u0 += kTile * UPL) {
#pragma unroll
    for (int g = 0; g < kTile; g += kGroup) {
      T x[kGroup][UPL];
#pragma unroll
      for (int q = 0; q < kGroup; q++) {
        const int sl = lane_base + g + q;
        const int kd = __shfl(kind, sl);
        const uint8_t* sp = reinterpret_cast<const uint8_t*>(__shfl((unsigned long long)src, sl));
#pragma unroll
        for (int w = 0; w < UPL; w++) {
          const uint32_t u = u0 + j + w * kTile;
          x[q][w] = T{};
          if (u < units) {
            if (kd == 2) x[q][w] = ld_unit<VEC, true>(sp, u);
            if (kd == 1) x[q][w] = ld_unit<VEC, false>(sp, u);
          }
        }
      }
#pragma unroll
      for (int q = 0; q < kGroup; q++) {
        const int sl = lane_base + g + q;
        const int kd = __shfl(kind, sl);
        uint8_t* dp = reinterpret_cast<uint8_t*>(__shfl((unsigned long long)dst, sl));
#pragma unroll
        for (int w = 0; w < UPL; w++) {
          const uint32_t u = u0 + j + w * kTile;
          if (u < units && kd) st_unit<VEC, false>(dp, u, x[q][w]);
        }
      }
    }
  }
}

/*
 * Rare path of the writers: lanes whose first probe met a LOCKED candidate, or
 * whose hit changed hands, get a coherent second probe by their tile.
 * On return `reprobe` is cleared for every lane whose bucket held no LOCKED
 * candidate, `hit` is the key's slot or -1, and (em_lo, em_hi) is the fresh
 * 128-bit mask of EMPTY digests.  Every lane of the wavefront must call this.
 */
constexpr int kMaxLockedWaits = 64;
__device__ __forceinline__ void settle_reprobes(const View& v, uint64_t key, uint32_t bkt,
                                                uint32_t digest, bool pending, bool& reprobe,
                                                int64_t& hit, uint64_t& em_lo, uint64_t& em_hi,
                                                int& waited, int lane) {
  const int tile = lane >> 3, j = lane & 7;
  const int lane_base = lane & ~(kTile - 1);
#pragma unroll 1
  for (int r = 0; r < kTile; r++) {
    const int src = lane_base + r;
    if (!__shfl((int)(pending && reprobe), src)) continue; /* tile-uniform */
    const uint64_t k2 = __shfl((unsigned long long)key, src);
    const uint32_t b2 = __shfl(bkt, src);
    const uint32_t d2 = __shfl(digest, src);
    uint32_t em16 = 0;
    const int64_t found = tile_reprobe(v, k2, b2, d2, tile, j, em16);
    uint64_t lo = 0, hi = 0;
#pragma unroll
    for (int q = 0; q < kTile; q++) {
      const uint64_t m = __shfl(em16, lane_base + q) & 0xFFFFu;
      if (q < 4)
        lo |= m << (16 * q);
      else
        hi |= m << (16 * (q - 4));
    }
    if (j == r) {
      if (found == -2 && ++waited < kMaxLockedWaits) {
        __builtin_amdgcn_s_sleep(2);
      } else {
        /* a slot that stays LOCKED this long is held by lock_keys, not by a
         * wavefront of this launch: the key is not there to be found (the
         * reference reads LOCKED as "another key", lookup_ptr.cuh:93-110) */
        hit = found == -2 ? -1 : found;
        reprobe = false;
        em_lo = lo;
        em_hi = hi;
      }
    }
  }
}

/*
 * LOCKED_RULE: the victim scan of the lock-key kernels used by the pointer
 * overload and by hybrid mode (find_ptr_or_insert.cuh:170-200,
 * upsert.cuh:1478-1524): slots whose key is LOCKED or EMPTY are invisible to
 * it.  Also used once lock_keys may have left LOCKED slots in the table, which
 * the plain scan would pick and wait for without end.  Whether a key is
 * refused at score == min is a separate switch (UpsertArgs::refuse_equal).
 */
/* WAVES wavefronts per workgroup, each with its own 64 keys and its own staging area.  One
 * everywhere except insert_and_evict on a table that is about full, whose wavefronts claim their
 * part of the evicted-keys output together: updates of one word are served one at a time, about
 * 15 ns each, and one per wavefront and trip (some 24 thousand for 2^20 keys into full buckets)
 * took 0.07 ms of the call's 0.46.  (While buckets have free slots there is nothing to claim,
 * and two wavefronts that wait for each other in every trip are 4 % slower than one.) */
template <int OP, int VEC, int UPL, bool LOCKED_RULE, bool BOUNDS = false, int WAVES = 1, bool HOLD = false>
__global__ void __launch_bounds__(kWave * WAVES)
    __attribute__((amdgpu_waves_per_eu(BOUNDS ? 4 : 1)))
upsert_kernel(View v, UpsertArgs a) {
  static_assert(!(BOUNDS && LOCKED_RULE), "the bounded search does not look at key words");
  static_assert(WAVES == 1 || OP == kOpInsertAndEvict, "only insert_and_evict has anything to share");
  static_assert(!HOLD || OP == kOpInsertOrAssign || OP == kOpFindOrInsert, "the calls with a hybrid form");
  __shared__ KeyMeta s_meta_all[WAVES][kWave];
  __shared__ int64_t s_slot_all[WAVES][kWave];
  __shared__ __attribute__((aligned(16))) uint16_t s_em_all[WAVES][kWave][kTile];
  __shared__ uint8_t s_unsure_all[WAVES][kWave];
  /* what the wavefronts of a workgroup tell each other in a trip (two sets, used in turn):
   * entries for the evicted-keys output and whether any key is still pending; then where the
   * workgroup's entries start */
  __shared__ uint32_t s_trip[2][WAVES];
  __shared__ unsigned long long s_claim[2];

  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  KeyMeta* const s_meta = s_meta_all[wave];
  int64_t* const s_slot = s_slot_all[wave];
  uint16_t (*const s_em)[kTile] = s_em_all[wave];
  uint8_t* const s_unsure = s_unsure_all[wave];
  const int tile = lane >> 3, j = lane & 7;
  const uint64_t i = ((uint64_t)blockIdx.x * WAVES + wave) * kWave + lane;
  const uint32_t units = v.value_bytes / VEC;

  uint64_t bound_cap = 0, bound_ceil = 0;
  if constexpr (BOUNDS) {
    bound_cap = a.bound_cap_in ? *a.bound_cap_in : a.bound_cap;
    if (a.bound_cap_out && blockIdx.x == 0 && threadIdx.x == 0) *a.bound_cap_out = now_ns(a.clock, 0);
    /* EpochLRU: the limit is a clock reading, the scores are made from it (kernel_utils.cuh:403-411) */
    if (a.strategy == HKV_EPOCH_LRU) bound_cap = (a.epoch << 32) | ((bound_cap >> 20) & kLow32);
    if (a.bound_ceil) {
      /* the word is raised to this call's limit by one thread while the others read it: either
       * value is one that no bound is above, the old bounds by the old value and the bounds this
       * call sets by its limit */
      const uint64_t c = *a.bound_ceil;
      bound_ceil = c > bound_cap ? c : bound_cap;
      if (blockIdx.x == 0 && threadIdx.x == 0 && bound_cap > c) *a.bound_ceil = bound_cap;
    }
  }
  const uint64_t key = stage_keys(v, a.keys, a.n, i, s_meta, s_slot, lane);
  const uint64_t in_score = (a.scores && i < a.n) ? a.scores[i] : 0;
  s_unsure[lane] = 0;
  __syncthreads();
  probe_wave<true, kTwoStepWriters>(v, s_meta, s_slot, s_em, s_unsure, lane);
  __syncthreads();

  /* ---- state of the key this lane owns ---------------------------------------------- */
  const KeyMeta me = s_meta[lane];
  const uint32_t digest = me.info & 0xFFu;
  const uint32_t start = me.info >> 16;
  const uint64_t bslot = (uint64_t)me.bkt * kBucketSize;
  int64_t hit = s_slot[lane];
  uint64_t em_lo, em_hi;
  {
    const uint4 e = *reinterpret_cast<const uint4*>(s_em[lane]);
    em_lo = e.x | ((uint64_t)e.y << 32);
    em_hi = e.z | ((uint64_t)e.w << 32);
  }
  bool pending = (me.info & 0x100u) != 0;
  bool reprobe = pending && hit < 0 && s_unsure[lane];
  int waited = 0;

  /* The trip loop is controlled by a wavefront-uniform value only: all 64
   * lanes take part in every trip (the tile-cooperative steps read registers
   * of lanes whose own key is already done), until no lane is pending. */
  unsigned long long pend_mask = __ballot(pending);
  /* with several wavefronts per workgroup all of them make as many trips as the slowest, so
   * that every one arrives at the workgroup's barriers */
  bool more = pend_mask != 0;
  if constexpr (WAVES > 1) more = __syncthreads_or(more);
  /* HOLD: hybrid mode, insert_or_assign and find_or_insert: the slots of a batch stay LOCKED to
   * the end of the launch (an instantiation of its own: as a run-time switch it cost the kernels
   * of tables without host rows 3 %) */
  constexpr bool hold = HOLD;
  /* Where every slot that is taken stays LOCKED to the end of the launch, a LOCKED word is never
   * this key's slot about to be given back: it is another key of the batch, or this key on its
   * way out.  The second probe does not wait for it.  (With the waits, a key whose digest
   * matched a held slot kept its wavefront alive for 64 rounds: 0.15 ms per 2^20 keys.) */
  if (HOLD || (OP == kOpFindOrInsertPtr && a.locked_key_ptrs != nullptr)) waited = kMaxLockedWaits;
  for (int trip = 0; more; trip++) {
    if (__ballot(pending && reprobe))
      settle_reprobes(v, key, me.bkt, digest, pending, reprobe, hit, em_lo, em_hi, waited, lane);

    bool active = pending && !reprobe;
    if constexpr (OP == kOpAccumOrAssign) {
      /* accum_or_assign.cuh:139-156: a key whose flag and presence disagree (accumulate onto
       * a key that is not there, assign to one that is) changes nothing.  It is done without
       * a lock: the reference takes the slot and gives it back, and a free slot that is given
       * back has meanwhile been crossed off by the bucket's other new keys, which then look
       * for a victim in a bucket that is not full. */
      if (active && (a.accum_flags[i] != 0) != (hit >= 0)) {
        pending = false;
        active = false;
      }
    }
    const uint64_t desired = desired_when_missed(a, in_score, i);
    int got = kStNone;
    uint32_t pos = 0;
    uint64_t victim = 0;

    /* what the key needs, known from the probe: its own slot, a free one, or a victim's */
    const bool has_hit = active && hit >= 0;
    const bool has_free = active && hit < 0 && (em_lo | em_hi) != 0;
    const bool want_scan = active && hit < 0 && (em_lo | em_hi) == 0;

    /* ---- step 1: full buckets: min-score search by the tile, before any lock is taken ------------
     * (the search holds nothing, so the keys that were found wait for nobody while it runs, and
     * the locks of all 64 keys are then taken in one round trip; two buckets in flight per tile
     * in the full scan took 32 more registers and with them a wavefront per SIMD: 0.308 against
     * 0.323 ms per 2^20 keys) */
    uint64_t best = kMaxScore;
    uint32_t bpos = 0;
    uint64_t new_bound = 0;
    if constexpr (BOUNDS) {
      /* the bounds of four buckets, then the most promising score line of each, in flight */
      const uint32_t need = tile_ballot(want_scan, tile);
      const int lane_base = lane & ~(kTile - 1);
#pragma unroll
      for (int h = 0; h < kTile; h += 4) {
        if (!__ballot(((need >> h) & 0xFu) != 0)) continue;
        uint64_t bs[4], bd[4];
        uint32_t g[4];
        uint4 x[4];
#pragma unroll
        for (int q = 0; q < 4; q++) {
          bs[q] = __shfl((unsigned long long)bslot, lane_base + h + q);
          bd[q] = kMaxScore;
          if ((need >> (h + q)) & 1u) bd[q] = ld_u64(v.bounds + (bs[q] >> 4) + j);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
          uint64_t b = bd[q];
          uint32_t gi = (uint32_t)j;
          tile_min_pair(b, gi);
          g[q] = gi;
          x[q] = make_uint4(0, 0, 0, 0);
          if ((need >> (h + q)) & 1u) x[q] = line_load(v, bs[q], g[q], j);
        }
#pragma unroll
        for (int q = 0; q < 4; q++) {
          if ((need >> (h + q)) & 1u) {
            uint64_t b0, nb0;
            uint32_t p0;
            bounded_min(v, bs[q], tile, j, bd[q], g[q], x[q], bound_cap, b0, p0, nb0);
            if (j == h + q) {
              best = b0;
              bpos = p0;
              new_bound = nb0;
            }
          }
        }
      }
    } else {
      uint32_t need = tile_ballot(want_scan, tile);
      const int lane_base = lane & ~(kTile - 1);
      for (unsigned long long more = __ballot(need != 0); more; more = __ballot(need != 0)) {
        if (need) {
          const int r0 = __ffs(need) - 1;
          need &= need - 1;
          const uint64_t bs0 = __shfl((unsigned long long)bslot, lane_base + r0);
          uint64_t sc0[2 * kTile];
          uint64_t kc0[LOCKED_RULE ? 2 * kTile : 1];
          scan_load<LOCKED_RULE>(v, bs0, j, sc0, kc0);
          uint64_t b0;
          uint32_t p0;
          scan_reduce<LOCKED_RULE>(v, sc0, kc0, j, b0, p0);
          if (j == r0) {
            best = b0;
            bpos = p0;
          }
        }
      }
    }

    /* ---- step 2: one lock attempt per key, all in flight together ----------------------------------
     * a compare-and-swap for a key that was found (key -> LOCKED) or that takes a free slot
     * (EMPTY -> LOCKED: the first free slot at or after the key's start position, so that keys
     * of one bucket spread over the free slots); an exchange for a victim: whatever key the slot
     * held is the victim and the slot is locked (instead of a load and a compare-and-swap).
     * LOCKED coming back means somebody else holds the slot (nothing changed); EMPTY means
     * the slot is free after all and is now this key's. */
    bool refused_now = false;
    bool try_victim = false;
    if (want_scan) {
      if (a.refuse_equal ? (desired <= best) : (desired < best)) {
        refused_now = true;
        got = kStRefused;
      } else {
        try_victim = true;
      }
    }
    uint32_t p_free = 0;
    if (has_free) {
      p_free = first_from(em_lo, em_hi, start);
      if (p_free < 64)
        em_lo &= ~(UINT64_C(1) << p_free);
      else
        em_hi &= ~(UINT64_C(1) << (p_free - 64));
    }
    uint64_t seen = has_hit ? key : v.empty_key;
    bool cas_ok = false;
    if (has_hit || has_free)
      cas_ok = cas_lock(has_hit ? v.keys + hit : v.keys + bslot + p_free, seen, v.locked_key);
    uint64_t* const kp = v.keys + bslot + bpos;
    uint64_t vk = v.locked_key;
    if (try_victim) vk = swap_lock(kp, v.locked_key);

    /* ---- step 3: what came back ------------------------------------------------------------------------ */
    if (has_hit) {
      if (cas_ok) {
        got = kStDuplicate;
        pos = (uint32_t)(hit - (int64_t)bslot);
        victim = key;
      } else {
        /* The slot belongs to another key now (ours was evicted in this batch, or the probe
         * was looking at somebody else's lock), or it is LOCKED: by a key of this batch that is
         * taking it over or about to give it back, or for good (lock_keys, a batch-mate of
         * the pointer overload that keeps its slots).  The second probe finds out which,
         * and its waiting is bounded. */
        hit = -1;
        reprobe = true;
      }
    }
    if (has_free) {
      if (cas_ok) {
        got = kStEmpty;
        pos = p_free;
        victim = v.empty_key;
      }
      /* somebody else took it: up to two more of the bucket's free slots */
#pragma unroll 1
      for (int attempt = 1; attempt < 3 && got == kStNone && (em_lo | em_hi); attempt++) {
        const uint32_t p = first_from(em_lo, em_hi, start);
        if (p < 64)
          em_lo &= ~(UINT64_C(1) << p);
        else
          em_hi &= ~(UINT64_C(1) << (p - 64));
        uint64_t e = v.empty_key;
        if (cas_lock(v.keys + bslot + p, e, v.locked_key)) {
          got = kStEmpty;
          pos = p;
          victim = v.empty_key;
        }
      }
    }
    if (try_victim) {
      const bool mine = vk != v.locked_key && vk != v.empty_key;
      if (vk == v.empty_key) {
        /* The slot has become free since the probe (an erase that runs beside this call) and
         * the exchange has locked it: it is taken like any free slot.  Putting EMPTY back and
         * searching again would find the same slot, whose old score is still the lowest. */
        got = kStEmpty;
        pos = bpos;
        victim = v.empty_key;
      }
      if (mine) {
        /* somebody may have raised the score since the search */
        if (ld_u64(v.scores + bslot + bpos) <= best) {
          victim = vk;
          got = (vk == v.reclaim_key) ? kStReclaimed : kStEvict;
          pos = bpos;
        } else {
          st_unlock(kp, vk); /* nothing was written under this lock */
        }
      } /* else: the victim is locked or was taken by somebody else; next trip */
    }

    /* ---- step 4: critical sections of every lock taken in this trip ------------------------------ */
    const bool locked = got != kStNone && got != kStRefused;
    const uint64_t slot = bslot + pos;
    uint8_t* row = value_row(v, slot);
    const bool commit = locked;

    /* upsert_and_evict.cuh:188-194, 218-224, 236-245: an evicted key leaves with its old row
     * and the scanned minimum, a refused key with its input.  One counter update per workgroup
     * and trip: every wavefront posts its number of entries (and whether it has keys left for
     * another trip, which is known by now), the first wavefront claims the sum, and the
     * bookkeeping stores of the trip go out while that update is under way. */
    const bool emit = OP == kOpInsertAndEvict && (refused_now || (commit && got == kStEvict));
    unsigned long long votes = 0, claimed = 0;
    uint32_t before = 0, total = 0;
    const int set = trip & 1;
    if (OP == kOpInsertAndEvict) {
      votes = __ballot(emit);
      const bool stay = __ballot(pending && got == kStNone) != 0;
      if (lane == 0) s_trip[set][wave] = (uint32_t)__popcll(votes) | (stay ? 0x100u : 0u);
      __syncthreads();
      more = false;
#pragma unroll
      for (int w = 0; w < WAVES; w++) {
        const uint32_t t = s_trip[set][w];
        if (w < wave) before += t & 0xFFu;
        total += t & 0xFFu; /* the same in every wavefront of the workgroup */
        more |= (t & 0x100u) != 0;
      }
      if (total && threadIdx.x == 0) claimed = atomicAdd(a.evicted_counter, (unsigned long long)total);
    }
    if (OP == kOpFindOrInsertPtr && (locked || refused_now)) {
      a.out_ptrs[i] = locked ? row : nullptr;
      a.founds[i] = got == kStDuplicate;
      if (a.locked_key_ptrs) a.locked_key_ptrs[i] = locked ? v.keys + slot : nullptr;
    }
    if (commit) {
      /* a victim's slot gets a score of this call: what bounds its line now is the lowest of
       * the line's other scores */
      if (BOUNDS && (got == kStEvict || got == kStReclaimed))
        st_u64(v.bounds + (slot >> 4), new_bound < bound_cap ? new_bound : bound_cap);
      const uint64_t stored = write_meta(v, a, slot, digest, desired, in_score, i, got != kStDuplicate, hold);
      if (hold) {
        /* hybrid mode: the slots of a batch stay LOCKED until all its keys are settled; the
         * list starts out as all null */
        a.locked_key_ptrs[i] = v.keys + slot;
        a.held_scores[i] = stored;
      }
      /* Scores from the caller may be below what the line's bound says: a key that goes into a
       * free slot, and a key that was found, under Customized (its score becomes the caller's)
       * and under EpochLFU (it moves to the epoch of today, which may be an earlier one than its
       * own; LFU only adds to it).  Such a key lowers the bound itself.  A key that takes a
       * victim's slot cannot be below the victim's score, which the bound was not above, except
       * under LFU, whose line has just been given a bound that no score of this call is below. */
      if (BOUNDS && a.bound_ceil && stored < bound_ceil &&
          (got == kStEmpty ||
           (got == kStDuplicate && (a.strategy == HKV_CUSTOMIZED || a.strategy == HKV_EPOCH_LFU))))
        __hip_atomic_fetch_min(v.bounds + (slot >> 4), stored, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (OP == kOpInsertAndEvict && total) {
      if (threadIdx.x == 0) s_claim[set] = claimed;
      __syncthreads();
      if (votes) {
        const unsigned long long idx = s_claim[set] + before + __popcll(votes & ((1ull << lane) - 1));
        if (emit) {
          a.evicted_keys[idx] = refused_now ? key : victim;
          if (a.evicted_scores) a.evicted_scores[idx] = refused_now ? desired : best;
        }
        bulk_evicted<VEC, UPL>(emit ? (refused_now ? 1 : 2) : 0,
                               refused_now ? a.values_in + i * v.value_bytes : row,
                               a.evicted_values + idx * v.value_bytes, units, lane);
      }
    }
    if (OP != kOpFindOrInsertPtr) {
      int move = kMoveNone;
      uint8_t* usr = nullptr;
      if (commit) {
        if (OP == kOpInsertOrAssign || OP == kOpInsertAndEvict) {
          move = kMoveInToTable;
          usr = const_cast<uint8_t*>(a.values_in) + i * v.value_bytes;
        } else if (OP == kOpFindOrInsert) {
          move = got == kStDuplicate ? kMoveTableToIo : kMoveInToTable;
          usr = a.values_io + i * v.value_bytes;
        } else if (OP == kOpAccumOrAssign) {
          move = got == kStDuplicate ? kMoveAccum : kMoveInToTable;
          usr = const_cast<uint8_t*>(a.values_in) + i * v.value_bytes;
        }
      }
      if (__ballot(move != kMoveNone))
        bulk_rows<VEC, UPL, OP == kOpFindOrInsert, OP == kOpAccumOrAssign>(
            move, row, usr, units, a.value_kind, lane);
    }

    /* ---- step 5: everything written under the locks is out; release them --------------------------- */
    wait_stores();
    /* the pointer overload may be asked to leave its slots locked for unlock_keys; the upserts
     * of hybrid mode leave theirs locked until the launch is over */
    const bool keep_locked = HOLD || (OP == kOpFindOrInsertPtr && a.locked_key_ptrs != nullptr);
    if (locked && !keep_locked) st_unlock(v.keys + slot, commit ? key : victim);
    if (keep_locked) {
      const unsigned long long kept = __ballot(locked);
      /* (no count where the launch that follows opens the slots again: one word takes one update
       * at a time, and a wavefront's worth of them per trip is a quarter of a millisecond per
       * 2^20 keys) */
      if (a.locked_count && kept && lane == (int)__ffsll(kept) - 1)
        atomicAdd(locked_shard(a.locked_count), (unsigned long long)__popcll(kept));
    }
    if (got != kStNone) pending = false;
    pend_mask = __ballot(pending);
    if constexpr (WAVES == 1) more = pend_mask != 0;
  }
}

/* ---- assign family: update keys that are present, never insert -----------------
 * The score rule is ScoreFunctor::update_without_missed (kernel_utils.cuh:
 * 304-321, 373-392, 436-453, 519-557, 594-612).  Without the group lock several
 * updaters may run at once, and a batch may repeat a key: then the row changes under
 * the slot lock (LOCKFREE == false). */

struct AssignArgs {
  const uint64_t* keys;
  const uint8_t* values; /* null: scores only */
  const uint64_t* scores;
  uint64_t n;
  uint64_t epoch;
  Clock clock;
  int32_t touch_scores;
  int32_t strategy;
  /* Customized and EpochLFU tables with score bounds in use: the device word no bound is above (as
   * UpsertArgs::bound_ceil); a key whose new score is below it lowers its line's bound */
  const unsigned long long* bound_ceil;
};

/* the score the slot holds afterwards; kMaxScore when it was left as it is */
__device__ __forceinline__ uint64_t assign_score(const View& v, const AssignArgs& a,
                                                 uint64_t slot, uint64_t i) {
  const int STRATEGY = a.strategy;
  uint64_t s;
  if (STRATEGY == HKV_LRU) {
    s = now_ns(a.clock, i);
  } else if (STRATEGY == HKV_LFU) {
    if (!a.scores) return kMaxScore;
    s = ld_u64(v.scores + slot) + a.scores[i];
  } else if (STRATEGY == HKV_EPOCH_LRU) {
    s = (a.epoch << 32) | ((now_ns(a.clock, i) >> 20) & kLow32);
  } else if (STRATEGY == HKV_EPOCH_LFU) {
    if (!a.scores) return kMaxScore;
    const uint64_t in = a.scores[i] & kLow32;
    s = ld_u64(v.scores + slot) & kLow32;
    if (kLow32 - s > in)
      s += (a.epoch << 32) | in;
    else
      s = (a.epoch << 32) | kLow32;
  } else {
    if (!a.scores) return kMaxScore;
    s = a.scores[i];
  }
  st_u64(v.scores + slot, s);
  return s;
}

/* LOCKFREE: the call is the only writer on the table while it runs and its keys are unique,
 * so every slot it touches has one owner and the slot lock (one compare-and-swap and one
 * unlock store per key, each a read-modify-write at the memory side) is left out:
 * assign at capacity 2^26, dim 64: 0.215 -> 0.185 ms per 2^20 keys. */
template <int VEC, int UPL, bool LOCKFREE>
__global__ void __launch_bounds__(kWave)
assign_kernel(View v, AssignArgs a) {
  __shared__ KeyMeta s_meta[kWave];
  __shared__ int64_t s_slot[kWave];
  __shared__ uint8_t s_unsure[kWave];
  const int lane = threadIdx.x;
  const uint64_t i = (uint64_t)blockIdx.x * kWave + lane;
  const uint32_t units = v.value_bytes / VEC;
  const uint64_t bound_ceil = a.bound_ceil ? *a.bound_ceil : 0;
  const uint64_t key = stage_keys(v, a.keys, a.n, i, s_meta, s_slot, lane);
  s_unsure[lane] = 0;
  __syncthreads();
  probe_wave<true, kTwoStepWriters>(v, s_meta, s_slot, nullptr, s_unsure, lane);
  __syncthreads();
  const KeyMeta me = s_meta[lane];
  int64_t hit = s_slot[lane];
  bool reprobe = hit < 0 && s_unsure[lane];
  bool pending = (me.info & 0x100u) && (hit >= 0 || reprobe);
  int waited = 0;
  uint64_t em_lo = 0, em_hi = 0;
  unsigned long long pend_mask = __ballot(pending);
  while (pend_mask) {
    if (__ballot(pending && reprobe))
      settle_reprobes(v, key, me.bkt, me.info & 0xFFu, pending, reprobe, hit, em_lo, em_hi, waited, lane);
    int got = kStNone;
    if (pending && !reprobe) {
      if (hit < 0) {
        got = kStAbsent;
      } else {
        uint64_t seen = key;
        if (LOCKFREE || cas_lock(v.keys + hit, seen, v.locked_key)) {
          got = kStDuplicate;
        } else {
          /* the slot changed hands or is LOCKED (another updater for a moment, lock_keys for
           * good): look again, for a bounded time */
          hit = -1;
          reprobe = true;
        }
      }
    }
    const bool locked = got == kStDuplicate;
    uint8_t* row = value_row(v, (uint64_t)(hit < 0 ? 0 : hit));
    if (locked && a.touch_scores) {
      const uint64_t stored = assign_score(v, a, (uint64_t)hit, i);
      if (a.bound_ceil && stored < bound_ceil)
        __hip_atomic_fetch_min(v.bounds + ((uint64_t)hit >> 4), stored, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    if (a.values) {
      const int move = locked ? kMoveInToTable : kMoveNone;
      uint8_t* usr = const_cast<uint8_t*>(a.values) + i * v.value_bytes;
      if (__ballot(move != kMoveNone))
        bulk_rows<VEC, UPL, false, false>(move, row, usr, units, 0, lane);
    }
    if (!LOCKFREE) {
      wait_stores();
      if (locked) st_unlock(v.keys + hit, key);
    }
    if (got != kStNone) pending = false;
    pend_mask = __ballot(pending);
    if (pend_mask) __builtin_amdgcn_s_sleep(1);
  }
}

}  // namespace hkv
#endif
