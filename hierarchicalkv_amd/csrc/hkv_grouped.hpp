/*
 * Two-phase insert_or_assign: the path behind hkv_insert_or_assign_noalloc, the entry point for
 * callers that cannot allocate.
 *
 * Same per-key semantics as the slot-lock kernel (hkv_upsert.hpp, after upsert.cuh:52-233);
 * what changes is who may touch a slot.  An inserter runs alone on the table (the API-level
 * group lock, as group_lock.cuh:43-56), so the only conflicts are between keys of the same
 * batch, and only between keys that are absent: a key that is present owns its slot (keys of a
 * batch are unique), absent keys of one bucket compete for its free slots and victims.  Hence
 * two phases, each one kernel:
 *
 *   upsert_hits_kernel   every key is probed as in find.  A key that is present
 *                        gets its new score and row at once, without a lock.
 *                        An absent key is hung into the list of its bucket:
 *                        one exchange on the bucket's head word (a 4-byte-per-
 *                        bucket array that stays in the last-level cache), and
 *                        the previous head goes into next[i], which is written
 *                        for all 64 keys of the wavefront in one coalesced line.
 *   chained_miss_kernel  one lane per bucket reads (and clears) the head word
 *                        and walks the list; each bucket that has keys is then
 *                        owned by one 8-lane tile, which reads the digest line
 *                        once and the 128 scores once, places its keys one
 *                        after the other there (free slot, else minimum score,
 *                        ties to the lowest slot) and writes the digest line
 *                        back whole.
 *
 * The serial order this amounts to - all present keys, then the absent ones
 * bucket by bucket - is one of the orders the slot-lock kernel could have
 * produced.  The path has no locks and needs no memory beyond the list heads and links, which is
 * why the no-alloc entry point runs on it; as the general path it measured slower than the
 * slot-lock kernel (two launches, a second pass over the keys), so nothing else uses it.
 */
#ifndef HKV_GROUPED_HPP_
#define HKV_GROUPED_HPP_

#include "hkv_upsert.hpp"

namespace hkv {

constexpr int kGrpKeys = 2;       /* keys of one bucket handled per pass of a tile */
constexpr int kChainStage = 4;    /* keys of one bucket staged per walk of its list */
constexpr uint32_t kChainEnd = 0; /* head / next hold key index + 1 */

/* ---- register-resident bucket state ------------------------------------------------ */

/* byte `p` (0..15) of the 16 digest bytes a lane holds; selects and shifts
 * only, so that the four words stay in registers */
__device__ __forceinline__ uint32_t dg_byte(const uint4& d, uint32_t p) {
  const uint32_t a = (p & 8u) ? d.z : d.x;
  const uint32_t b = (p & 8u) ? d.w : d.y;
  const uint32_t x = (p & 4u) ? b : a;
  return (x >> ((p & 3u) * 8)) & 0xFFu;
}
__device__ __forceinline__ void dg_set(uint4& d, uint32_t p, uint32_t byte) {
  const uint32_t sh = (p & 3u) * 8;
  const uint32_t clr = 0xFFu << sh, put = byte << sh;
  const uint32_t w = p >> 2;
  const uint32_t c0 = w == 0 ? clr : 0u, c1 = w == 1 ? clr : 0u, c2 = w == 2 ? clr : 0u,
                 c3 = w == 3 ? clr : 0u;
  d.x = (d.x & ~c0) | (put & c0);
  d.y = (d.y & ~c1) | (put & c1);
  d.z = (d.z & ~c2) | (put & c2);
  d.w = (d.w & ~c3) | (put & c3);
}

/* ScoreFunctor<Strategy>::update_with_digest (kernel_utils.cuh:291-302,
 * 353-371, 422-434, 490-517, 581-593) as a value: the score an accepted key
 * leaves in its slot; false when the score stays as it is. */
__device__ __forceinline__ bool final_score(const UpsertArgs& a, bool new_insert, uint64_t desired,
                                            uint64_t in_score, uint64_t old, uint64_t& s) {
  const int STRATEGY = a.strategy;
  s = desired;
  if (STRATEGY == HKV_LFU) {
    if (!a.scores) return false;
    s = new_insert ? in_score : in_score + old;
  } else if (STRATEGY == HKV_EPOCH_LFU) {
    if (!new_insert) {
      s = old & kLow32;
      if (kLow32 - s > (desired & kLow32))
        s += desired;
      else
        s = (desired & kEpochMask) | kLow32;
    }
  }
  return true;
}

/* The lists of absent keys, one per bucket: head[bucket] is the batch index + 1 of the key
 * hung in last (0: none), next[i] the index + 1 of the key hung in before key i.  head[] is
 * all zero between calls: the second phase clears what it reads. */
struct ChainArgs {
  uint32_t* head;       /* [buckets_num] */
  uint32_t* next;       /* [n] */
  uint32_t locked_rule; /* refuse when score <= min, not < (upsert.cuh:1478-1524) */
};

/*
 * Phase 1.  One wavefront per 64 keys, as lookup_kernel: probe, then
 *   present  new score (update_with_digest with the slot's old score where the
 *            strategy needs it) and the row traffic of the operation, the whole
 *            wavefront moving the rows of its keys, VEC bytes per lane;
 *   absent   hung into the list of its bucket for the second phase.
 */
template <int VEC>
__global__ void __launch_bounds__(kWave)
upsert_hits_kernel(View v, UpsertArgs a, ChainArgs h) {
  __shared__ KeyMeta s_meta[kWave];
  __shared__ int64_t s_slot[kWave];
  const int lane = threadIdx.x;
  const uint64_t base = (uint64_t)blockIdx.x * kWave;
  const uint64_t i = base + lane;
  stage_keys(v, a.keys, a.n, i, s_meta, s_slot, lane);
  const uint64_t in_score = (a.scores && i < a.n) ? a.scores[i] : 0;
  __syncthreads();
  probe_wave<false, true>(v, s_meta, s_slot, nullptr, nullptr, lane);
  __syncthreads();

  const bool valid = (s_meta[lane].info & 0x100u) != 0;
  const int64_t slot = s_slot[lane];
  const bool hit = valid && slot >= 0;
  const bool miss = valid && slot < 0;
  if (i < a.n) {
    uint32_t before = kChainEnd;
    if (miss)
      before = __hip_atomic_exchange(h.head + s_meta[lane].bkt, (uint32_t)i + 1, __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
    h.next[i] = before;
  }
  if (hit) {
    const uint64_t desired = desired_when_missed(a, in_score, i);
    const bool needs_old = a.strategy == HKV_LFU || a.strategy == HKV_EPOCH_LFU;
    const uint64_t old = needs_old ? v.scores[slot] : 0;
    uint64_t snew;
    if (final_score(a, false, desired, in_score, old, snew)) v.scores[slot] = snew;
  }
  /* rows: 64 rows x units-per-row spread over the 64 lanes; all loads of a
   * batch are issued before the first store */
  using T = typename VecType<VEC>::type;
  const uint32_t units = v.value_bytes / VEC;
  const uint32_t total = units * kWave;
  const bool pow2 = (units & (units - 1)) == 0;
  const uint32_t sh = 31 - __clz(units);
  constexpr int kBatch = VEC == 16 ? 16 : 4;
  const uint8_t* usr_base = a.values_in + base * v.value_bytes;
  for (uint32_t idx0 = lane; idx0 < total; idx0 += kWave * kBatch) {
    T buf[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; b++) {
      const uint32_t idx = idx0 + b * kWave;
      buf[b] = T{};
      if (idx < total) {
        const uint32_t kk = pow2 ? (idx >> sh) : (idx / units);
        const uint32_t c = idx - kk * units;
        if (s_slot[kk] >= 0) buf[b] = ld_unit<VEC, false>(usr_base + (uint64_t)kk * v.value_bytes, c);
      }
    }
#pragma unroll
    for (int b = 0; b < kBatch; b++) {
      const uint32_t idx = idx0 + b * kWave;
      if (idx < total) {
        const uint32_t kk = pow2 ? (idx >> sh) : (idx / units);
        const uint32_t c = idx - kk * units;
        const int64_t sl = s_slot[kk];
        if (sl >= 0) st_unit<VEC, true>(value_row(v, (uint64_t)sl), c, buf[b]);
      }
    }
  }
}

/* ---- cross-lane moves inside an 8-lane tile without the LDS permute unit -------------------- */

/* value of the partner lane (lane ^ 1, lane ^ 2: data-parallel moves inside a
 * quad; lane ^ 4: one swizzle) */
__device__ __forceinline__ uint32_t xor1_u32(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0xB1, 0xF, 0xF, true); /* quad_perm [1,0,3,2] */
}
__device__ __forceinline__ uint32_t xor2_u32(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, 0x4E, 0xF, 0xF, true); /* quad_perm [2,3,0,1] */
}
__device__ __forceinline__ uint32_t xor4_u32(uint32_t x) {
  return (uint32_t)__builtin_amdgcn_ds_swizzle((int)x, 0x101F); /* and 0x1f, or 0, xor 4 */
}
/* (score, slot) pairs order by score, then by slot: the reference's sequential
 * scan with a strict '<' keeps the lowest slot among equal scores
 * (upsert.cuh:166-183) */
__device__ __forceinline__ bool pair_lt(uint64_t s, uint32_t p, uint64_t t, uint32_t q) {
  return s < t || (s == t && p < q);
}

/* The two smallest (score, slot) pairs of a bucket. */
struct Top2 {
  uint64_t s1, s2;
  uint32_t p1, p2;
};

constexpr uint32_t kNoSlot = 255;

/*
 * Scan of a bucket's 128 scores by the 8 lanes of a tile: lane j reads the
 * slots {16 it + 2 j, 16 it + 2 j + 1}, one coalesced 128-byte line per `it`
 * and tile, keeps its two smallest pairs, and three exchange steps merge the
 * lanes' pairs.  Slot `skip` does not take part (a slot a key of this pass has
 * just moved into: its score is still on its way).  Two pairs are enough for
 * a pass of two keys; the scores themselves are not kept, which is what keeps
 * the kernel's register count low.
 */
__device__ __forceinline__ Top2 tile_top2(const View& v, uint64_t bslot, int j, uint32_t skip) {
  uint4 raw[kTile];
#pragma unroll
  for (int it = 0; it < kTile; it++)
    raw[it] = *reinterpret_cast<const uint4*>(v.scores + bslot + it * 16 + j * 2);
  Top2 t;
  t.s1 = t.s2 = kMaxScore;
  t.p1 = t.p2 = kNoSlot;
#pragma unroll
  for (int q = 0; q < 2 * kTile; q++) {
    const uint4& r = raw[q >> 1];
    const uint64_t x = (q & 1) ? (r.z | ((uint64_t)r.w << 32)) : (r.x | ((uint64_t)r.y << 32));
    const uint32_t px = (q >> 1) * 16 + 2 * (uint32_t)j + (q & 1);
    if (px == skip) continue;
    if (pair_lt(x, px, t.s1, t.p1)) {
      t.s2 = t.s1;
      t.p2 = t.p1;
      t.s1 = x;
      t.p1 = px;
    } else if (pair_lt(x, px, t.s2, t.p2)) {
      t.s2 = x;
      t.p2 = px;
    }
  }
#define HKV_TOP2_STEP(FN)                                                                      \
  {                                                                                            \
    const uint64_t a1 = (uint64_t)FN((uint32_t)t.s1) | ((uint64_t)FN((uint32_t)(t.s1 >> 32)) << 32); \
    const uint64_t a2 = (uint64_t)FN((uint32_t)t.s2) | ((uint64_t)FN((uint32_t)(t.s2 >> 32)) << 32); \
    const uint32_t q1 = FN(t.p1), q2 = FN(t.p2);                                               \
    Top2 m;                                                                                    \
    if (pair_lt(a1, q1, t.s1, t.p1)) {                                                         \
      m.s1 = a1;                                                                               \
      m.p1 = q1;                                                                               \
      const bool second = pair_lt(a2, q2, t.s1, t.p1);                                         \
      m.s2 = second ? a2 : t.s1;                                                               \
      m.p2 = second ? q2 : t.p1;                                                               \
    } else {                                                                                   \
      m.s1 = t.s1;                                                                             \
      m.p1 = t.p1;                                                                             \
      const bool second = pair_lt(a1, q1, t.s2, t.p2);                                         \
      m.s2 = second ? a1 : t.s2;                                                               \
      m.p2 = second ? q1 : t.p2;                                                               \
    }                                                                                          \
    t = m;                                                                                     \
  }
  HKV_TOP2_STEP(xor1_u32)
  HKV_TOP2_STEP(xor2_u32)
  HKV_TOP2_STEP(xor4_u32)
#undef HKV_TOP2_STEP
  return t;
}

/*
 * Phase 2, one bucket: the absent keys of the batch that fall into bucket
 * `bkt` are the entries [sb, se) of the sorted LDS arrays.  Called by the 8
 * lanes of a tile together; `lane` is the lane inside the wavefront.  `dg` is
 * the lane's 16 bytes of the bucket's digest line.
 *
 * Everything that steers the work (which key goes where, what it displaces) is
 * computed by all 8 lanes alike from the same LDS entries, so the lanes agree
 * without talking; only the minimum search and the free-slot mask cross lanes.
 */
template <int VEC, int UPL>
__device__ __forceinline__ void group_bucket(const View& v, const UpsertArgs& a,
                                             const ChainArgs& g, uint32_t bkt, uint32_t sb,
                                             uint32_t se, const uint64_t* s_key,
                                             const uint32_t* s_idx, const uint32_t* s_info,
                                             uint32_t units, int lane, uint4 dg) {
  static_assert(kGrpKeys == 2, "tile_top2 serves a pass of two keys");
  const int j = lane & (kTile - 1);
  const int tile = lane >> 3;
  const int tile_base = lane & ~(kTile - 1);
  const uint64_t bslot = (uint64_t)bkt * kBucketSize;
  const uint8_t* rows_in = a.values_in;

  bool dg_dirty = false;

  /* free slots of the bucket, bit p for slot p */
  uint64_t em_lo = 0, em_hi = 0;
  {
    const uint32_t m16 = match16_natural(dg, v.empty_digest * 0x01010101u);
    if (tile_ballot(m16 != 0, tile)) {
#pragma unroll
      for (int q = 0; q < kTile; q++) {
        const uint64_t m = __shfl(m16, tile_base + q) & 0xFFFFu;
        if (q < 4)
          em_lo |= m << (16 * q);
        else
          em_hi |= m << (16 * (q - 4));
      }
    }
  }

  for (uint32_t q0 = sb; q0 < se; q0 += kGrpKeys) {
    const int mg = (int)(se - q0) < kGrpKeys ? (int)(se - q0) : kGrpKeys;
    /* a later pass may read what an earlier one wrote (a victim's key and row) */
    if (q0 != sb) wait_stores();

    /* ---- the rows the keys came with: asked for now, stored when the slot is known ------------ */
    constexpr bool kPre = VEC == 16 && UPL <= 2;
    using T = typename VecType<VEC>::type;
    T xin[kPre ? kGrpKeys : 1][kPre ? UPL : 1];
    if constexpr (kPre) {
#pragma unroll
      for (int q = 0; q < kGrpKeys; q++) {
        const uint8_t* us = rows_in + (uint64_t)s_idx[q < mg ? q0 + q : sb] * v.value_bytes;
#pragma unroll
        for (int w = 0; w < UPL; w++) {
          const uint32_t u = j + w * kTile;
          xin[q][w] = T{};
          if (q < mg && u < units) xin[q][w] = ld_unit<VEC, false>(us, u);
        }
      }
    }

    /* outcome of key q of the pass, the same in every lane of the tile */
    int got[kGrpKeys];
    uint32_t pos[kGrpKeys];
    uint64_t snew[kGrpKeys];
    bool wrs[kGrpKeys], cancelled[kGrpKeys], need_vk[kGrpKeys];
    int vic_from[kGrpKeys];
    bool scanned = false;
    Top2 top{};

    /* ---- the keys of the pass, one after the other -------------------------------------------------- */
#pragma unroll
    for (int q = 0; q < kGrpKeys; q++) {
      got[q] = kStNone;
      pos[q] = 0;
      snew[q] = 0;
      wrs[q] = false;
      cancelled[q] = false;
      need_vk[q] = false;
      vic_from[q] = -1;
      if (q >= mg) continue;
      const uint64_t kq = s_key[q0 + q];
      const uint64_t iq = s_idx[q0 + q];
      const uint32_t info = s_info[q0 + q];
      const uint64_t in_score = a.scores ? a.scores[iq] : 0;
      const uint64_t dq = desired_when_missed(a, in_score, iq);
      wrs[q] = final_score(a, true, dq, in_score, 0, snew[q]);
      /* the same key earlier in this pass (batches are meant to hold unique
       * keys): the first one wins, this one changes nothing */
      bool dup = false;
#pragma unroll
      for (int p = 0; p < q; p++)
        dup |= (got[p] == kStEmpty || got[p] == kStEvict) && s_key[q0 + p] == kq;
      if (dup) {
        got[q] = kStDuplicate;
        cancelled[q] = true;
        continue;
      }
      if (em_lo | em_hi) {
        const uint32_t p = first_from(em_lo, em_hi, (info >> 8) & 0x7Fu);
        if (p < 64)
          em_lo &= ~(UINT64_C(1) << p);
        else
          em_hi &= ~(UINT64_C(1) << (p - 64));
        got[q] = kStEmpty;
        pos[q] = p;
        if (j == (int)(p >> 4)) dg_set(dg, p & 15u, info & 0xFFu);
        dg_dirty = true;
        continue;
      }
      if (!scanned) {
        /* a key of this pass that has just taken the last free slot is not
         * part of the scan: it competes with its new score below */
        uint32_t skip = kNoSlot;
#pragma unroll
        for (int r = 0; r < q; r++)
          if (got[r] == kStEmpty) skip = pos[r];
        top = tile_top2(v, bslot, j, skip);
        scanned = true;
      }
      /* minimum over what the scan saw, less the slots this pass has already
       * taken over, plus the keys this pass has placed */
      uint64_t best = kMaxScore;
      uint32_t bpos = kNoSlot;
      {
        bool used1 = false, used2 = false;
#pragma unroll
        for (int r = 0; r < q; r++) {
          if (got[r] == kStEvict) {
            used1 |= pos[r] == top.p1;
            used2 |= pos[r] == top.p2;
          }
        }
        if (!used1 && pair_lt(top.s1, top.p1, best, bpos)) {
          best = top.s1;
          bpos = top.p1;
        }
        if (!used2 && pair_lt(top.s2, top.p2, best, bpos)) {
          best = top.s2;
          bpos = top.p2;
        }
#pragma unroll
        for (int r = 0; r < q; r++) {
          if ((got[r] == kStEmpty || got[r] == kStEvict) && !cancelled[r] && wrs[r] &&
              pair_lt(snew[r], pos[r], best, bpos)) {
            best = snew[r];
            bpos = pos[r];
          }
        }
      }
      const bool refuse = g.locked_rule ? (dq <= best) : (dq < best);
      if (refuse) {
        got[q] = kStRefused;
        continue;
      }
      /* the slot may belong to a key of this very pass (one that has just been
       * inserted with a low score): that key's writes are dropped, it leaves
       * through the eviction */
#pragma unroll
      for (int p = 0; p < q; p++) {
        if (!cancelled[p] && pos[p] == bpos && (got[p] == kStEmpty || got[p] == kStEvict)) {
          cancelled[p] = true;
          vic_from[q] = p;
        }
      }
      /* kStReclaimed is told apart from kStEvict by the key word, which is read
       * only when somebody needs it: a tombstone always carries the tombstone digest */
      const bool tomb_digest =
          tile_ballot(j == (int)(bpos >> 4) && dg_byte(dg, bpos & 15u) == v.reclaim_digest, tile) != 0;
      got[q] = kStEvict;
      need_vk[q] = vic_from[q] < 0 && tomb_digest;
      pos[q] = bpos;
      if (j == (int)(bpos >> 4)) dg_set(dg, bpos & 15u, info & 0xFFu);
      dg_dirty = true;
    }

    /* ---- victims: live key or tombstone ------------------------------------------------------------- */
    uint64_t victim[kGrpKeys];
#pragma unroll
    for (int q = 0; q < kGrpKeys; q++) {
      victim[q] = 0;
      if (got[q] == kStEvict && need_vk[q]) victim[q] = v.keys[bslot + pos[q]];
    }
#pragma unroll
    for (int q = 0; q < kGrpKeys; q++) {
      if (got[q] == kStEvict && need_vk[q] && victim[q] == v.reclaim_key) {
        got[q] = kStReclaimed;
      }
    }

    /* ---- key, score, row of every key that stays -------------------------------------------------------- */
#pragma unroll
    for (int q = 0; q < kGrpKeys; q++) {
      const bool writes =
          (got[q] == kStEmpty || got[q] == kStReclaimed || got[q] == kStEvict) && !cancelled[q];
      if (!writes) continue;
      const uint64_t slot = bslot + pos[q];
      if (j == 0) {
        v.keys[slot] = s_key[q0 + q];
        if (wrs[q]) v.scores[slot] = snew[q];
      }
      uint8_t* tb = value_row(v, slot);
      if constexpr (kPre) {
#pragma unroll
        for (int w = 0; w < UPL; w++) {
          const uint32_t u = j + w * kTile;
          if (u < units) st_unit<VEC, true>(tb, u, xin[q][w]);
        }
      } else {
        const uint8_t* us = rows_in + (uint64_t)s_idx[q0 + q] * v.value_bytes;
        for (uint32_t u0 = 0; u0 < units; u0 += kTile * UPL) {
          T x[UPL];
#pragma unroll
          for (int w = 0; w < UPL; w++) {
            const uint32_t u = u0 + j + w * kTile;
            x[w] = T{};
            if (u < units) x[w] = ld_unit<VEC, false>(us, u);
          }
#pragma unroll
          for (int w = 0; w < UPL; w++) {
            const uint32_t u = u0 + j + w * kTile;
            if (u < units) st_unit<VEC, true>(tb, u, x[w]);
          }
        }
      }
    }
  }

  if (dg_dirty) st_u128(v.digests + bslot + j * 16, dg);
}

/*
 * Phase 2.  One wavefront per 64 consecutive buckets.
 *   walk   lane L reads the head word of bucket 64 w + L, clears it, and follows the list:
 *          up to kChainStage keys go to the lane's part of the LDS staging arrays (key,
 *          batch index, digest and start slot); the 64 lists are walked side by side, one
 *          memory round trip per step for the whole wavefront;
 *   place  the buckets that have keys are dealt out to the 8 tiles in turn; a tile works
 *          through its buckets with group_bucket, the digest line of its next bucket being
 *          asked for before the current one is worked on.
 * A list longer than kChainStage is finished in further rounds of walk and place.
 */
template <int VEC, int UPL>
__global__ void __launch_bounds__(kWave)
__attribute__((amdgpu_waves_per_eu(3)))
chained_miss_kernel(View v, UpsertArgs a, ChainArgs g) {
  __shared__ uint64_t s_key[kWave * kChainStage];
  __shared__ uint32_t s_idx[kWave * kChainStage];
  __shared__ uint32_t s_info[kWave * kChainStage]; /* digest | start << 8 */
  __shared__ uint8_t s_count[kWave];
  __shared__ uint8_t s_list[kWave]; /* lanes (buckets) that have keys in this pass */

  const int lane = threadIdx.x;
  const int tile = lane >> 3, j = lane & (kTile - 1);
  const uint64_t b0 = (uint64_t)blockIdx.x * kWave;
  const uint64_t my_bkt = b0 + lane;
  const uint32_t units = v.value_bytes / VEC;

  uint32_t h = kChainEnd;
  if (my_bkt < v.buckets_num) {
    h = g.head[my_bkt];
    if (h != kChainEnd) g.head[my_bkt] = kChainEnd;
  }
  bool again = false;
  while (__ballot(h != kChainEnd)) {
    /* a further round re-reads digest lines and scores that the round before has written */
    const bool again_round = again;
    if (again) {
      wait_stores();
      __syncthreads();
    }
    again = true;
    /* ---- walk -------------------------------------------------------------------------------- */
    int cnt = 0;
    while (__ballot(h != kChainEnd && cnt < kChainStage)) {
      if (h != kChainEnd && cnt < kChainStage) {
        const uint32_t i = h - 1;
        const uint64_t key = a.keys[i];
        h = g.next[i];
        uint32_t bkt, start, digest;
        locate(v, key, bkt, start, digest);
        const int at = lane * kChainStage + cnt;
        s_key[at] = key;
        s_idx[at] = i;
        s_info[at] = digest | (start << 8);
        cnt++;
      }
    }
    s_count[lane] = (uint8_t)cnt;
    const unsigned long long have = __ballot(cnt > 0);
    if (cnt > 0) s_list[__popcll(have & ((1ull << lane) - 1))] = (uint8_t)lane;
    __syncthreads();

    /* ---- place -------------------------------------------------------------------------------- */
    const int nwork = __popcll(have);
    /* a round after the first reads lines that this wavefront has written: past the caches */
    const bool reread = again_round;
    auto digests_of = [&](int w) {
      const uint64_t bkt = b0 + s_list[w];
      if (reread) return ld_digests16(v, (uint32_t)bkt, j);
      return *reinterpret_cast<const uint4*>(v.digests + bkt * kBucketSize + j * 16);
    };
    int w0 = tile;
    uint4 dg0 = make_uint4(0, 0, 0, 0);
    if (w0 < nwork) dg0 = digests_of(w0);
    while (w0 < nwork) {
      const int w1 = w0 + kTilesPerWave;
      uint4 dg1 = make_uint4(0, 0, 0, 0);
      if (w1 < nwork) dg1 = digests_of(w1);
      const uint32_t lb = s_list[w0];
      const uint32_t sb = lb * kChainStage;
      group_bucket<VEC, UPL>(v, a, g, (uint32_t)(b0 + lb), sb, sb + s_count[lb], s_key, s_idx,
                                 s_info, units, lane, dg0);
      w0 = w1;
      dg0 = dg1;
    }
  }
}

}  // namespace hkv
#endif
