/*
 * The upsert family: insert_or_assign, insert_and_evict, find_or_insert
 * (values and pointers), accum_or_assign.  One kernel template for every
 * load factor; one 64-lane wavefront per workgroup, 64 keys per wavefront.
 *
 * Replaces tlp_v1/tlp_v2/pipeline_upsert_kernel_with_io (upsert.cuh:27-986),
 * the *_upsert_and_evict_kernel_unique kernels (upsert_and_evict.cuh:27-1099),
 * the find_or_insert kernels (find_or_insert.cuh:27-1050), the pointer kernel
 * (find_ptr_or_insert.cuh:27-246) and accum_or_assign_kernel_with_io
 * (accum_or_assign.cuh:83-174).  Per-key semantics follow upsert.cuh:52-233.
 *
 * Phase 1 (batched over the 64 keys): the probe of hkv_lookup.hpp, which also
 *   records where each bucket has EMPTY-looking digests.
 * Phase 2 (8 rounds, one key per 8-lane tile): take the slot lock with a
 *   64-bit CAS on the key word (key -> LOCKED for a hit, EMPTY -> LOCKED for a
 *   free slot, victim -> LOCKED after the min-score scan), write digest and
 *   score, move the value row with the tile, release the key word.
 *
 * The min-score scan reads the bucket's 128 scores as 8 coalesced 128-byte
 * lines per tile (16 scores per lane), reduces inside the lane and then over
 * the 8 lanes; ties go to the lowest slot, as in the reference's sequential
 * scan with a strict '<' (upsert.cuh:166-183).
 *
 * Lock discipline on a SIMD machine: a tile that has taken a lock finishes its
 * critical section in the same trip of the retry loop, and the loop's exit
 * test is a wavefront-wide ballot.  A tile that spins on a slot another tile
 * of the same wavefront holds therefore always finds it released on its next
 * trip.
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
  uint8_t* founds;
  uint64_t n;
  uint64_t epoch;
  Clock clock;
  int32_t value_kind;
  int32_t strategy; /* hkv_evict_strategy; uniform, so a scalar branch */
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
__device__ __forceinline__ void write_meta(const View& v, const UpsertArgs& a,
                                           uint64_t slot, uint32_t digest,
                                           uint64_t desired, uint64_t in_score,
                                           uint64_t i, bool new_insert) {
  const int STRATEGY = a.strategy;
  uint64_t s = desired;
  if (STRATEGY == HKV_LRU) {
    s = now_ns(a.clock, i);
  } else if (STRATEGY == HKV_LFU) {
    if (!a.scores) return;
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
  st_u8(v.digests + slot, (uint8_t)digest);
  st_u64(v.scores + slot, s);
}

/* dst[e] += delta[e] on a table row, element type by KIND
 * (accum_or_assign_vector, accum_or_assign.cuh:24-35).  The row is read and
 * written coherently: another key of the batch may have written it. */
template <int KIND>
__device__ __forceinline__ void tile_accum(uint8_t* row, const uint8_t* delta,
                                           uint32_t bytes, int j) {
  if (KIND == HKV_VALUE_F32) {
    uint32_t* d = reinterpret_cast<uint32_t*>(row);
    const float* s = reinterpret_cast<const float*>(delta);
    for (uint32_t e = j; e < bytes / 4; e += kTile)
      st_u32(d + e, __float_as_uint(__uint_as_float(ld_u32(d + e)) + s[e]));
  } else if (KIND == HKV_VALUE_F64) {
    uint64_t* d = reinterpret_cast<uint64_t*>(row);
    const double* s = reinterpret_cast<const double*>(delta);
    for (uint32_t e = j; e < bytes / 8; e += kTile)
      st_u64(d + e, (uint64_t)__double_as_longlong(__longlong_as_double((long long)ld_u64(d + e)) + s[e]));
  } else if (KIND == HKV_VALUE_I32) {
    uint32_t* d = reinterpret_cast<uint32_t*>(row);
    const uint32_t* s = reinterpret_cast<const uint32_t*>(delta);
    for (uint32_t e = j; e < bytes / 4; e += kTile) st_u32(d + e, ld_u32(d + e) + s[e]);
  } else {
    uint64_t* d = reinterpret_cast<uint64_t*>(row);
    const uint64_t* s = reinterpret_cast<const uint64_t*>(delta);
    for (uint32_t e = j; e < bytes / 8; e += kTile) st_u64(d + e, ld_u64(d + e) + s[e]);
  }
}

/* float rows that allow 16-byte access on the caller's side: 8 table bytes
 * (two floats) per coherent access */
__device__ __forceinline__ void tile_accum_f32x4(uint8_t* row,
                                                 const uint8_t* delta,
                                                 uint32_t bytes, int j) {
  uint64_t* d = reinterpret_cast<uint64_t*>(row);
  const float4* s = reinterpret_cast<const float4*>(delta);
  for (uint32_t u = j; u < bytes / 16; u += kTile) {
    const uint64_t lo = ld_u64(d + 2 * u), hi = ld_u64(d + 2 * u + 1);
    const float4 y = s[u];
    const float x0 = __uint_as_float((uint32_t)lo) + y.x;
    const float x1 = __uint_as_float((uint32_t)(lo >> 32)) + y.y;
    const float x2 = __uint_as_float((uint32_t)hi) + y.z;
    const float x3 = __uint_as_float((uint32_t)(hi >> 32)) + y.w;
    st_u64(d + 2 * u, __float_as_uint(x0) | ((uint64_t)__float_as_uint(x1) << 32));
    st_u64(d + 2 * u + 1, __float_as_uint(x2) | ((uint64_t)__float_as_uint(x3) << 32));
  }
}

enum : int {
  kStInitial = 0,
  kStDuplicate = 1,
  kStEmpty = 2,
  kStReclaimed = 3,
  kStEvict = 4,
  kStRefused = 5,
  kStSkip = 6
};

/*
 * LOCKED_RULE: behaviour of the lock-key kernels used by the pointer overload
 * and by hybrid mode (find_ptr_or_insert.cuh:170-200, upsert.cuh:1478-1524):
 * slots whose key is LOCKED or EMPTY are invisible to the victim scan and a
 * key is refused when score <= min instead of score < min.
 */
template <int OP, int VEC, bool LOCKED_RULE>
__global__ void __launch_bounds__(kWave)
upsert_kernel(View v, UpsertArgs a) {
  __shared__ KeyMeta s_meta[kWave];
  __shared__ int64_t s_slot[kWave];
  __shared__ uint64_t s_in_score[kWave];
  __shared__ uint32_t s_emask[kTile][kWave];
  __shared__ uint8_t s_unsure[kWave];

  const int lane = threadIdx.x;
  const int tile = lane >> 3, j = lane & 7;
  const uint64_t base = (uint64_t)blockIdx.x * kWave;
  {
    const uint64_t i = base + lane;
    stage_keys(v, a.keys, a.n, i, s_meta, s_slot, lane);
    s_in_score[lane] = (a.scores && i < a.n) ? a.scores[i] : 0;
    s_unsure[lane] = 0;
  }
  __syncthreads();
  probe_wave<true>(v, s_meta, s_slot, s_emask, s_unsure, lane);
  __syncthreads();

#pragma unroll 1
  for (int r = 0; r < kTile; r++) {
    const int kk = r * kTile + tile;
    const uint64_t i = base + kk;
    const KeyMeta m = s_meta[kk];
    const uint64_t key = m.key;
    const uint32_t digest = m.info & 0xFFu;
    const uint32_t start = m.info >> 16;
    const uint64_t bslot = (uint64_t)m.bkt * kBucketSize;
    const uint64_t in_score = s_in_score[kk];
    int64_t hit = s_slot[kk];
    uint32_t em = s_emask[r][lane];
    int status = (m.info & 0x100u) ? kStInitial : kStSkip;
    bool reprobe = hit < 0 && s_unsure[kk];

    while (true) {
      if (status == kStInitial && reprobe) {
        const int64_t found = tile_reprobe(v, key, m.bkt, digest, tile, j, em);
        if (found == -2) {
          __builtin_amdgcn_s_sleep(2);
        } else {
          hit = found;
          reprobe = false;
        }
      } else if (status == kStInitial) {
        uint64_t desired = desired_when_missed(a, in_score, i);
        int got = kStInitial;   /* outcome if a lock was taken in this trip */
        uint32_t pos = 0;
        uint64_t victim = 0;
        uint64_t min_score = 0;

        if (hit >= 0) {
          /* 1 = locked by us, 0 = held by another tile (try again), -1 = the
           * slot now belongs to another key: ours was evicted in this batch */
          int ok = 0;
          if (j == 0) {
            uint64_t seen = key;
            if (cas_lock(v.keys + hit, seen, v.locked_key))
              ok = 1;
            else if (seen != v.locked_key)
              ok = -1;
          }
          ok = tile_bcast(ok, tile, 0);
          if (ok > 0) {
            got = kStDuplicate;
            pos = (uint32_t)(hit - (int64_t)bslot);
            victim = key;
          } else if (ok < 0) {
            /* the slot belongs to another key now: ours was evicted in this
             * batch, or the probe was looking at somebody else's lock */
            hit = -1;
            reprobe = true;
          } else {
            __builtin_amdgcn_s_sleep(2);
          }
        } else {
          const uint32_t lanes = tile_ballot(em != 0, tile);
          if (lanes) {
            /* free slot: start with the lane that covers the key's start
             * position so keys of one bucket spread over the free slots */
            const int s4 = (int)(start >> 4);
            const uint32_t rot = ((lanes >> s4) | (lanes << (kTile - s4))) & 0xFFu;
            const int jl = ((__ffs(rot) - 1) + s4) & 7;
            const uint32_t eml = tile_bcast(em, tile, jl);
            const uint32_t p = (uint32_t)jl * 16 + bw_to_pos(__ffs(eml) - 1);
            bool ok = false;
            if (j == 0) {
              uint64_t seen = v.empty_key;
              ok = cas_lock(v.keys + bslot + p, seen, v.locked_key);
            }
            ok = tile_bcast(ok, tile, 0);
            if (j == jl) em &= em - 1;
            if (ok) {
              got = kStEmpty;
              pos = p;
              victim = v.empty_key;
            }
          } else {
            /* full bucket: minimum over the 128 scores */
            uint64_t best = kMaxScore;
            uint32_t bpos = 0;
            uint64_t sc[2 * kTile];
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
                const uint64_t ka = ld_u64(kp), kb = ld_u64(kp + 1);
                if (ka == v.locked_key || ka == v.empty_key) sc[2 * it] = kMaxScore;
                if (kb == v.locked_key || kb == v.empty_key) sc[2 * it + 1] = kMaxScore;
              }
            }
#pragma unroll
            for (int it = 0; it < kTile; it++) {
              const uint32_t p0 = it * 16 + j * 2;
              if (sc[2 * it] < best) {
                best = sc[2 * it];
                bpos = p0;
              }
              if (sc[2 * it + 1] < best) {
                best = sc[2 * it + 1];
                bpos = p0 + 1;
              }
            }
#pragma unroll
            for (int off = 1; off < kTile; off <<= 1) {
              const uint64_t ob = __shfl_xor(best, off);
              const uint32_t op = __shfl_xor(bpos, off);
              if (ob < best || (ob == best && op < bpos)) {
                best = ob;
                bpos = op;
              }
            }
            min_score = best;
            const bool refuse = LOCKED_RULE ? (desired <= best) : (desired < best);
            if (refuse) {
              status = kStRefused;
              if (OP == kOpInsertAndEvict) {
                /* upsert_and_evict.cuh:188-194, 243-245 */
                unsigned long long idx = 0;
                if (j == 0) idx = atomicAdd(a.evicted_counter, 1ull);
                idx = tile_bcast(idx, tile, 0);
                if (j == 0) {
                  a.evicted_keys[idx] = key;
                  if (a.evicted_scores) a.evicted_scores[idx] = desired;
                }
                tile_copy<VEC, false, false>(a.evicted_values + idx * v.value_bytes,
                                             a.values_in + i * v.value_bytes,
                                             v.value_bytes, j);
              }
              if (OP == kOpFindOrInsertPtr && j == 0) {
                a.out_ptrs[i] = nullptr;
                a.founds[i] = 0;
              }
            } else {
              int ok = 0;
              uint64_t vk = 0;
              if (j == 0) {
                uint64_t* kp = v.keys + bslot + bpos;
                vk = ld_u64(kp);
                uint64_t seen = vk;
                if (vk != v.locked_key && vk != v.empty_key &&
                    cas_lock(kp, seen, v.locked_key)) {
                  /* somebody may have raised the score since the scan */
                  if (ld_u64(v.scores + bslot + bpos) <= best)
                    ok = 1;
                  else
                    st_unlock(kp, vk); /* nothing was written under this lock */
                }
              }
              ok = tile_bcast(ok, tile, 0);
              if (ok) {
                victim = tile_bcast(vk, tile, 0);
                got = (victim == v.reclaim_key) ? kStReclaimed : kStEvict;
                pos = bpos;
              } else {
                __builtin_amdgcn_s_sleep(2);
              }
            }
          }
        }

        if (got != kStInitial) {
          /* critical section: the slot's key word holds LOCKED */
          const uint64_t slot = bslot + pos;
          uint8_t* row = value_row(v, slot);
          bool commit = true;
          if (OP == kOpAccumOrAssign) {
            /* accum_or_assign.cuh:139-156: flag and outcome must agree */
            const bool is_accum = a.accum_flags[i] != 0;
            commit = is_accum == (got == kStDuplicate);
          }
          if (commit) {
            if (OP == kOpInsertAndEvict && got == kStEvict) {
              /* upsert_and_evict.cuh:218-224, 236-238: the old row leaves
               * before the new one lands */
              unsigned long long idx = 0;
              if (j == 0) idx = atomicAdd(a.evicted_counter, 1ull);
              idx = tile_bcast(idx, tile, 0);
              if (j == 0) {
                a.evicted_keys[idx] = victim;
                if (a.evicted_scores) a.evicted_scores[idx] = min_score;
              }
              tile_copy<VEC, false, true>(a.evicted_values + idx * v.value_bytes, row,
                                          v.value_bytes, j);
            }
            if (j == 0) {
              write_meta(v, a, slot, digest, desired, in_score, i,
                                   got != kStDuplicate);
              if (got == kStEmpty || got == kStReclaimed)
                atomicAdd(v.sizes + m.bkt, 1);
            }
            if (OP == kOpInsertOrAssign || OP == kOpInsertAndEvict) {
              tile_copy<VEC, true, false>(row, a.values_in + i * v.value_bytes,
                                          v.value_bytes, j);
            } else if (OP == kOpFindOrInsert) {
              uint8_t* user = a.values_io + i * v.value_bytes;
              if (got == kStDuplicate)
                tile_copy<VEC, false, true>(user, row, v.value_bytes, j);
              else
                tile_copy<VEC, true, false>(row, user, v.value_bytes, j);
            } else if (OP == kOpAccumOrAssign) {
              const uint8_t* user = a.values_in + i * v.value_bytes;
              if (got == kStDuplicate) {
                if (a.value_kind == HKV_VALUE_F32) {
                  if (VEC == 16)
                    tile_accum_f32x4(row, user, v.value_bytes, j);
                  else
                    tile_accum<HKV_VALUE_F32>(row, user, v.value_bytes, j);
                } else if (a.value_kind == HKV_VALUE_F64) {
                  tile_accum<HKV_VALUE_F64>(row, user, v.value_bytes, j);
                } else if (a.value_kind == HKV_VALUE_I32) {
                  tile_accum<HKV_VALUE_I32>(row, user, v.value_bytes, j);
                } else {
                  tile_accum<HKV_VALUE_I64>(row, user, v.value_bytes, j);
                }
              } else {
                tile_copy<VEC, true, false>(row, user, v.value_bytes, j);
              }
            } else if (OP == kOpFindOrInsertPtr) {
              if (j == 0) {
                a.out_ptrs[i] = row;
                a.founds[i] = got == kStDuplicate;
              }
            }
          }
          wait_stores();
          if (j == 0) st_unlock(v.keys + slot, commit ? key : victim);
          status = got;
        }
      }
      if (__ballot(status == kStInitial) == 0) break;
    }
  }
}

}  // namespace hkv
#endif
