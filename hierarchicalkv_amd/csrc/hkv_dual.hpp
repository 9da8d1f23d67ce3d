/*
 * Dual-bucket mode (TableMode::kMemory): every key has two candidate buckets,
 * b1 from the low hash word and b2 from the high one, and the digest is the top
 * hash byte (dual_bucket_utils.cuh:36-101).  Only insert_or_assign and find
 * run on such a table, as in the reference (merlin_hashtable.cuh:1166-1190,
 * 2483-2494); the other calls are refused by the host side.
 *
 * insert_or_assign replaces dual_bucket_pipeline_upsert_kernel_with_io
 * (dual_bucket_upsert.cuh:49-600): one 8-lane tile per key, eight keys per
 * wavefront, slot locks as in single-bucket mode.
 *   phase 0  the key is looked for in b1, then in b2 (digest match, key compare,
 *            CAS key -> LOCKED);
 *   phase 1  otherwise the bucket with fewer keys is tried first (b1 on a tie),
 *            then the other: the first EMPTY slot in circular order from the
 *            bucket's own start position is locked;
 *   phase 2  otherwise the minimum score over both buckets decides: the key is
 *            refused when its score is below it, else the slot holding the
 *            minimum is locked (b1 when min1 <= min2), its score is checked
 *            again under the lock and the attempt repeats when it moved or the
 *            slot was held by another tile.
 * A tile holds at most one lock, and finishes with it (row written, key word released)
 * at the place where it took it.
 *
 * find replaces dual_bucket_pipeline_lookup_kernel_with_io
 * (dual_bucket_lookup.cuh:25-140): lookup_kernel probes b1 for the 64 keys of
 * a wavefront, then b2 for those not found there.
 */
#ifndef HKV_DUAL_HPP_
#define HKV_DUAL_HPP_

#include "hkv_upsert.hpp"

namespace hkv {

/* how often phase 2 looks again before the key is given up as refused (every
 * repeat means another tile changed one of the two buckets in between) */
constexpr int kDualMaxTries = 1024;

template <int VEC>
__global__ void __launch_bounds__(kWave)
dual_upsert_kernel(View v, UpsertArgs a) {
  const int lane = threadIdx.x, tile = lane >> 3, j = lane & 7;
  const uint64_t i = (uint64_t)blockIdx.x * kTilesPerWave + tile;
  if (i >= a.n) return; /* the 8 lanes of a tile leave together */
  const uint64_t key = a.keys[i];
  if (is_reserved_key(v, key)) return;
  const uint64_t in_score = a.scores ? a.scores[i] : 0;
  const DualLoc L = locate_dual(v, key);
  const uint64_t desired = desired_when_missed(a, in_score, i);
  const uint32_t pat = L.digest * 0x01010101u;
  const uint32_t epat = v.empty_digest * 0x01010101u;

  uint4 dg[2];
  dg[0] = ld_digests16(v, L.bkt[0], j);
  dg[1] = ld_digests16(v, L.bkt[1], j);

  int64_t slot = -1;
  bool is_new = false, grew = false;

  /* phase 0: present in b1 or b2? */
#pragma unroll
  for (int w = 0; w < 2; w++) {
    if (slot >= 0) continue;
    uint32_t m = match16(dg[w], pat);
    uint64_t* kb = v.keys + (uint64_t)L.bkt[w] * kBucketSize + j * 16;
    int hit = -1;
    while (m) {
      const uint32_t p = bw_to_pos(__ffs(m) - 1);
      m &= m - 1;
      if (ld_u64(kb + p) != key) continue;
      uint64_t expect = key;
      if (cas_lock(kb + p, expect, v.locked_key)) {
        hit = (int)p;
        break;
      }
    }
    const uint32_t hits = tile_ballot(hit >= 0, tile);
    if (hits) {
      const int jl = __ffs(hits) - 1;
      slot = (int64_t)L.bkt[w] * kBucketSize + jl * 16 + tile_bcast(hit, tile, jl);
    }
  }

  /* phase 1: an EMPTY slot, the emptier bucket first */
  if (slot < 0) {
    const int32_t sz0 = (int32_t)ld_u32(reinterpret_cast<const uint32_t*>(v.sizes + L.bkt[0]));
    const int32_t sz1 = (int32_t)ld_u32(reinterpret_cast<const uint32_t*>(v.sizes + L.bkt[1]));
    const int first = sz0 <= sz1 ? 0 : 1;
#pragma unroll
    for (int turn = 0; turn < 2; turn++) {
      const int w = turn == 0 ? first : 1 - first;
      if (slot >= 0) continue;
      if ((w == 0 ? sz0 : sz1) >= (int32_t)kBucketSize) continue;
      const uint32_t em = match16_natural(w == 0 ? dg[0] : dg[1], epat);
      uint64_t lo = 0, hi = 0;
#pragma unroll
      for (int q = 0; q < kTile; q++) {
        const uint64_t e = tile_bcast(em, tile, q);
        if (q < 4)
          lo |= e << (16 * q);
        else
          hi |= e << (16 * (q - 4));
      }
      const uint32_t bkt = w == 0 ? L.bkt[0] : L.bkt[1];
      const uint32_t start = w == 0 ? L.start[0] : L.start[1];
      while (lo | hi) {
        const uint32_t p = first_from(lo, hi, start);
        int ok = 0;
        if (j == 0) {
          uint64_t expect = v.empty_key;
          ok = cas_lock(v.keys + (uint64_t)bkt * kBucketSize + p, expect, v.locked_key) ? 1 : 0;
          /* counted at once, not when the row is in: the other keys in flight choose their
           * bucket by these counters, and a stale count sends them to the fuller one */
          if (ok) atomicAdd(v.sizes + bkt, 1);
        }
        ok = tile_bcast(ok, tile, 0);
        if (ok) {
          slot = (int64_t)bkt * kBucketSize + p;
          is_new = true;
          break;
        }
        if (p < 64)
          lo &= ~(UINT64_C(1) << p);
        else
          hi &= ~(UINT64_C(1) << (p - 64));
      }
    }
  }

  /* The critical section of the lock this tile holds: digest and score, the row, and the
   * release of the key word.  It runs right where the lock was taken, before any tile of this
   * wavefront goes round the retry loop below again: a tile that still looks for a victim may
   * be waiting for exactly this lock, and lanes that have left a loop do not run again until
   * the other lanes have left it too. */
  auto commit = [&](int64_t at) {
    if (j == 0) {
      write_meta(v, a, (uint64_t)at, L.digest, desired, in_score, i, is_new);
      if (grew) atomicAdd(v.sizes + ((uint64_t)at >> 7), 1);
    }
    tile_copy<VEC, true, false>(value_row(v, (uint64_t)at),
                                a.values_in + i * (uint64_t)v.value_bytes, v.value_bytes, j);
    wait_stores();
    if (j == 0) st_unlock(v.keys + at, key);
  };
  bool pending = true;
  if (slot >= 0) {
    commit(slot);
    pending = false; /* no return here: the order of this block and the loop below must not be
                        left to the compiler's layout of two independent branches */
  }

  /* phase 2: the minimum score of both buckets.  The scan reads scores only: a slot that
   * another tile holds shows the score it had (it is retried until the tile has released it
   * with its new score), so the outcome is that of handling the keys one after the other in
   * some order. */
  for (int tries = 0; tries < kDualMaxTries && __ballot(pending) != 0; tries++) {
    int ok = 0; /* 1: a key is evicted, 2: the slot was free or a tombstone */
    uint64_t vs = 0;
    if (pending) {
      uint64_t best[2];
      uint32_t pos[2];
#pragma unroll
      for (int w = 0; w < 2; w++) {
        uint64_t sc[2 * kTile], kc[1];
        scan_load<false>(v, (uint64_t)L.bkt[w] * kBucketSize, j, sc, kc);
        scan_reduce<false>(v, sc, kc, j, best[w], pos[w]);
      }
      const int w = best[0] <= best[1] ? 0 : 1;
      const uint64_t mn = w == 0 ? best[0] : best[1];
      if (desired < mn) {
        pending = false; /* refused */
      } else {
        vs = (uint64_t)(w == 0 ? L.bkt[0] : L.bkt[1]) * kBucketSize + (w == 0 ? pos[0] : pos[1]);
        if (j == 0) {
          const uint64_t vk = swap_lock(v.keys + vs, v.locked_key);
          if (vk == v.locked_key) {
            /* held by another tile; look again */
          } else if (vk == v.empty_key) {
            ok = 2; /* freed or never filled: an insert into a free slot after all */
          } else if (ld_u64(v.scores + vs) <= mn) {
            ok = vk == v.reclaim_key ? 2 : 1;
          } else {
            st_unlock(v.keys + vs, vk); /* the score moved: not the minimum any more */
          }
        }
        ok = tile_bcast(ok, tile, 0);
      }
    }
    if (ok) {
      is_new = true;
      grew = ok == 2;
      commit((int64_t)vs);
      pending = false;
    }
    /* the loop is left by all lanes of the wavefront together, so the commit above is never
     * deferred to a point after the loop */
    if (__ballot(pending) == 0) break;
    __builtin_amdgcn_s_sleep(1);
  }
  /* still pending here: given up and treated as refused (the buckets kept changing under
   * kDualMaxTries looks) */
}

}  // namespace hkv
#endif
