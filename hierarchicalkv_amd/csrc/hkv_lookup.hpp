/*
 * Read-only lookups: find (value copy), find* (row pointer), contains, and
 * the missed-keys variant of find.  One 64-lane wavefront per workgroup,
 * 64 keys per wavefront.
 *
 * Replaces lookup_kernel_with_io_pipeline_v1 (lookup.cuh:119-378),
 * lookup_ptr_kernel_with_pipeline / tlp_lookup_ptr_kernel_with_filter
 * (lookup_ptr.cuh:25-374) and the contains kernels (contains.cuh:46-216).
 * No slot locks are taken: the API-level group lock keeps writers out, as in
 * the reference (group_lock.cuh:43-56).
 *
 * Phases of a wavefront
 *   own    lane L loads key L, hashes it and stages (key, bucket, digest) in LDS;
 *   probe  tile t (8 lanes) probes key 8t+r in round r = 0..7: lane j loads
 *          16 of the 128 digest bytes, so a tile reads one whole 128-byte line
 *          per round; the 8 rounds are issued back to back so 8 KB of digests
 *          are in flight per wavefront;
 *   verify every digest match is checked against the 8-byte key, the first
 *          lane's candidates first and the others only if those were not it;
 *          the hit slot goes to LDS;
 *   copy   the whole wavefront copies the found rows, VEC bytes per lane,
 *          so the output side is written in fully coalesced 1 KB pieces.
 */
#ifndef HKV_LOOKUP_HPP_
#define HKV_LOOKUP_HPP_

#include <type_traits>

#include "hkv_common.hpp"

namespace hkv {

struct FindArgs {
  const uint64_t* keys;
  uint8_t* out_values;     /* find */
  void** out_ptrs;         /* find* */
  uint8_t* founds;         /* may be null for the missed-keys variant */
  uint64_t* out_scores;    /* optional */
  uint64_t* missed_keys;   /* missed-keys variant */
  int32_t* missed_indices;
  int32_t* missed_size;
  uint64_t n;
};

/*
 * Probe the 64 keys staged in s_meta.  On return (after the caller's barrier)
 * s_slot[k] is the table slot of key k or -1.  WRITER selects the writers'
 * probe, which runs while other wavefronts change the table:
 *   - s_em[k][j] (when given) receives lane j's 16-bit mask of EMPTY digests of
 *     key k's bucket, bit p for byte 16j+p, so the 8 masks of a key read back
 *     as one 128-bit mask in slot order;
 *   - a candidate slot whose key word reads LOCKED may be this very key under
 *     another tile's lock, so s_unsure[k] is raised and the writer settles the
 *     question with a second, coherent probe of its own (tile_reprobe).
 */
template <bool WRITER, bool TWO_STEP>
__device__ __forceinline__ void probe_wave(const View& v, const KeyMeta* s_meta,
                                           int64_t* s_slot,
                                           uint16_t (*s_em)[kTile],
                                           uint8_t* s_unsure, int lane) {
  const int tile = lane >> 3, j = lane & 7;
  uint4 dg[kTile];
  uint32_t bkt[kTile];
  uint32_t inf[kTile];
#pragma unroll
  for (int r = 0; r < kTile; r++) {
    const KeyMeta m = s_meta[tile * kTile + r];
    bkt[r] = m.bkt;
    inf[r] = m.info;
    dg[r] = make_uint4(0, 0, 0, 0);
    if (m.info & 0x100u)
      dg[r] = *reinterpret_cast<const uint4*>(v.digests + (uint64_t)m.bkt * kBucketSize + j * 16);
  }
  /* TWO_STEP: candidates are verified in two steps.  An 8-byte key load costs a whole
   * 128-byte line of memory traffic, a key that is present has one true candidate, and a
   * false 8-bit match turns up in every second bucket: so step 1 fetches only the
   * candidates of one lane of the tile (a lane's 16 slots share one key line), the one
   * where the key most likely is, and the other lanes' candidates are fetched in step 2
   * only for the keys step 1 did not find: 1.03 to 1.27 key lines per key that is present
   * (keys that went into a free slot / into a victim's slot) instead of 1.44.  The lookups
   * and the kernels that move rows use it; erase and lock_keys, which move little besides
   * the probe and are bound by their dependent round trips, take all candidates at once. */
  uint32_t cm[kTile];    /* this lane's digest matches, bw order */
  uint32_t later[kTile]; /* lanes of the tile whose candidates wait for step 2 */
  uint64_t k0[kTile], k1[kTile];
#pragma unroll
  for (int r = 0; r < kTile; r++) {
    const bool valid = inf[r] & 0x100u;
    const uint32_t d = inf[r] & 0xFFu;
    cm[r] = valid ? match16(dg[r], d * 0x01010101u) : 0u;
    if (WRITER && s_em != nullptr)
      s_em[tile * kTile + r][j] =
          (uint16_t)(valid ? match16_natural(dg[r], v.empty_digest * 0x01010101u) : 0u);
    const uint32_t lanes = TWO_STEP ? tile_ballot(cm[r] != 0, tile) : 0u;
    /* step 1 takes the first lane with a candidate at or after the lane of the key's start
     * slot, going round: an insert takes the first free slot from there (the reference's
     * probe order, kernel_utils.cuh:636-643), so that is where the key most likely is */
    const uint32_t sl = inf[r] >> 20; /* start slot / 16 */
    const uint32_t turned = ((lanes >> sl) | (lanes << (kTile - sl))) & 0xFFu;
    const uint32_t first = (uint32_t)(__ffs(turned) - 1 + sl) & (kTile - 1);
    later[r] = lanes & ~(1u << first);
    const uint64_t* kb = v.keys + (uint64_t)bkt[r] * kBucketSize + j * 16;
    k0[r] = v.empty_key;
    k1[r] = v.empty_key;
    if (cm[r] && !((later[r] >> j) & 1u)) {
      k0[r] = kb[bw_to_pos(__ffs(cm[r]) - 1)];
      const uint32_t rest = cm[r] & (cm[r] - 1);
      if (rest) k1[r] = kb[bw_to_pos(__ffs(rest) - 1)];
    }
  }
  /* checks the candidates of this lane for key r against the fetched words (the third and
   * later candidates of a lane, rare, are loaded here) */
  auto check = [&](int r) {
    const int kk = tile * kTile + r;
    const uint64_t key = s_meta[kk].key;
    const uint64_t slot0 = (uint64_t)bkt[r] * kBucketSize + j * 16;
    uint32_t m = cm[r];
    int hit = -1;
    bool unsure = false;
    int c = 0;
    while (m) {
      const uint32_t p = bw_to_pos(__ffs(m) - 1);
      m &= m - 1;
      const uint64_t kx = c == 0 ? k0[r] : (c == 1 ? k1[r] : v.keys[slot0 + p]);
      c++;
      if (kx == key) {
        hit = (int)p;
        break;
      }
      if (WRITER && kx == v.locked_key) unsure = true;
    }
    if (hit >= 0)
      s_slot[kk] = (int64_t)(slot0 + hit);
    else if (WRITER && unsure)
      s_unsure[kk] = 1;
    return hit >= 0;
  };
  bool more = false;
#pragma unroll
  for (int r = 0; r < kTile; r++) {
    const bool mine = cm[r] && !((later[r] >> j) & 1u);
    const bool hit = mine && check(r);
    if (TWO_STEP) {
      if (tile_ballot(hit, tile)) later[r] = 0;
      more |= later[r] != 0;
    }
  }
  if (TWO_STEP && __ballot(more)) {
#pragma unroll
    for (int r = 0; r < kTile; r++) {
      if ((later[r] >> j) & 1u) {
        const uint64_t* kb = v.keys + (uint64_t)bkt[r] * kBucketSize + j * 16;
        k0[r] = kb[bw_to_pos(__ffs(cm[r]) - 1)];
        const uint32_t rest = cm[r] & (cm[r] - 1);
        if (rest) k1[r] = kb[bw_to_pos(__ffs(rest) - 1)];
      }
    }
#pragma unroll
    for (int r = 0; r < kTile; r++)
      if ((later[r] >> j) & 1u) check(r);
  }
}

/* the writers' probes (upsert and assign families): they move rows, like find */
constexpr bool kTwoStepWriters = true;

/* the 16 digest bytes of lane j of a tile, read past the caches */
__device__ __forceinline__ uint4 ld_digests16(const View& v, uint32_t bkt, int j) {
  const uint64_t off = (uint64_t)bkt * kBucketSize + j * 16;
  if (v.capacity < (UINT64_C(1) << 32)) return ld_u128_at(v.digests, v.capacity, off);
  const uint32_t* dp = reinterpret_cast<const uint32_t*>(v.digests + off);
  uint4 d;
  d.x = ld_u32(dp + 0);
  d.y = ld_u32(dp + 1);
  d.z = ld_u32(dp + 2);
  d.w = ld_u32(dp + 3);
  return d;
}

/*
 * Second opinion for a writer, by the 8-lane tile that owns the key, with
 * coherent loads: returns the slot of the key, -1 when the key is not in the
 * bucket, or -2 when a digest-matching slot is LOCKED right now (ask again).
 * `em` receives the lane's fresh mask of EMPTY digests (bit p for byte 16j+p).
 */
__device__ __forceinline__ int64_t tile_reprobe(const View& v, uint64_t key,
                                                uint32_t bkt, uint32_t digest,
                                                int tile, int j, uint32_t& em) {
  const uint4 d = ld_digests16(v, bkt, j);
  em = match16_natural(d, v.empty_digest * 0x01010101u);
  uint32_t m = match16(d, digest * 0x01010101u);
  const uint64_t slot0 = (uint64_t)bkt * kBucketSize + j * 16;
  int hit = -1;
  bool locked = false;
  while (m) {
    const uint32_t p = bw_to_pos(__ffs(m) - 1);
    m &= m - 1;
    const uint64_t kx = ld_u64(v.keys + slot0 + p);
    if (kx == key) {
      hit = (int)p;
      break;
    }
    if (kx == v.locked_key) locked = true;
  }
  const uint32_t hits = tile_ballot(hit >= 0, tile);
  const uint32_t locks = tile_ballot(locked, tile);
  if (hits) {
    const int jl = __ffs(hits) - 1;
    return (int64_t)tile_bcast((uint32_t)hit, tile, jl) + (int64_t)bkt * kBucketSize + jl * 16;
  }
  return locks ? -2 : -1;
}

/* Lane-owned part shared by all wave-per-64-keys kernels: load, hash, stage. */
__device__ __forceinline__ uint64_t stage_keys(const View& v,
                                               const uint64_t* keys, uint64_t n,
                                               uint64_t i, KeyMeta* s_meta,
                                               int64_t* s_slot, int lane) {
  uint64_t key = v.empty_key;
  if (i < n) key = keys[i];
  const bool valid = (i < n) && !is_reserved_key(v, key);
  uint32_t bkt = 0, start = 0, digest = 0;
  locate(v, key, bkt, start, digest);
  KeyMeta m;
  m.key = key;
  m.bkt = bkt;
  m.info = digest | (valid ? 0x100u : 0u) | (start << 16);
  s_meta[lane] = m;
  s_slot[lane] = -1;
  return key;
}

/* First pass of a dual-bucket find (dual_bucket_lookup.cuh:25-140): the keys
 * staged by stage_keys get their first bucket and the dual-mode digest. */
__device__ __forceinline__ void restage_first_bucket(const View& v, KeyMeta* s_meta, int lane) {
  KeyMeta m = s_meta[lane];
  if (m.info & 0x100u) {
    const DualLoc L = locate_dual(v, m.key);
    m.bkt = L.bkt[0];
    m.info = L.digest | 0x100u | (L.start[0] << 16);
    s_meta[lane] = m;
  }
}
/* Second pass of a dual-bucket find: the keys of the wavefront that b1 did not
 * hold are staged again with their second bucket; the others are switched off. */
__device__ __forceinline__ void restage_second_bucket(const View& v, KeyMeta* s_meta,
                                                      const int64_t* s_slot, int lane) {
  KeyMeta m = s_meta[lane];
  const bool again = (m.info & 0x100u) && s_slot[lane] < 0;
  if (again) {
    const DualLoc L = locate_dual(v, m.key);
    m.bkt = L.bkt[1];
    m.info = L.digest | 0x100u | (L.start[1] << 16);
  } else {
    m.info &= ~0x100u;
  }
  s_meta[lane] = m;
}


enum LookupMode { kLookupValues = 0, kLookupPtr = 1, kLookupContains = 2 };

/* WAVES wavefronts per workgroup, each with its own 64 keys and its own staging area.  One
 * wavefront per workgroup everywhere except the missed-keys variant, whose workgroups are
 * large so that the list of misses is claimed with one atomic per 1024 keys (updates of one
 * word are served one at a time, about 15 ns each: one per wavefront would take longer than
 * the lookup itself). */
template <int MODE, int VEC, bool DUAL = false, int WAVES = 1>
__global__ void __launch_bounds__(kWave * WAVES)
lookup_kernel(View v, FindArgs a) {
  __shared__ KeyMeta s_meta_all[WAVES][kWave];
  __shared__ int64_t s_slot_all[WAVES][kWave];
  __shared__ int32_t s_missed[2]; /* misses of the workgroup, start of its part of the list */
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  KeyMeta* const s_meta = s_meta_all[wave];
  int64_t* const s_slot = s_slot_all[wave];
  const uint64_t base = ((uint64_t)blockIdx.x * WAVES + wave) * kWave;
  const uint64_t i = base + lane;
  const uint64_t key = stage_keys(v, a.keys, a.n, i, s_meta, s_slot, lane);
  if (DUAL) restage_first_bucket(v, s_meta, lane);
  if (WAVES > 1 && threadIdx.x == 0) s_missed[0] = 0;
  __syncthreads();
  probe_wave<false, true>(v, s_meta, s_slot, nullptr, nullptr, lane);
  __syncthreads();
  if (DUAL) {
    restage_second_bucket(v, s_meta, s_slot, lane);
    __syncthreads();
    probe_wave<false, true>(v, s_meta, s_slot, nullptr, nullptr, lane);
    __syncthreads();
  }

  const int64_t my_slot = s_slot[lane];
  if (i < a.n) {
    if (a.founds) a.founds[i] = my_slot >= 0;
    if (my_slot >= 0) {
      if (a.out_scores) a.out_scores[i] = v.scores[my_slot];
      if (MODE == kLookupPtr) a.out_ptrs[i] = value_row(v, (uint64_t)my_slot);
    } else {
      if (MODE == kLookupPtr) a.out_ptrs[i] = nullptr;
    }
  }
  if (a.missed_size) {
    /* missed-keys variant (lookup.cuh:36-60): compact list of misses, in no particular
     * order; reserved keys are not probed and count as missed. */
    const bool miss = i < a.n && my_slot < 0;
    const unsigned long long mm = __ballot(miss);
    int32_t at = 0;
    if (WAVES > 1) {
      if (lane == 0 && mm) at = atomicAdd(&s_missed[0], (int32_t)__popcll(mm));
      __syncthreads();
      if (threadIdx.x == 0 && s_missed[0]) s_missed[1] = atomicAdd(a.missed_size, s_missed[0]);
      __syncthreads();
      at = __shfl(at, 0) + s_missed[1];
    } else {
      if (lane == 0 && mm) at = atomicAdd(a.missed_size, (int32_t)__popcll(mm));
      at = __shfl(at, 0);
    }
    if (miss) {
      at += (int32_t)__popcll(mm & ((1ull << lane) - 1));
      a.missed_keys[at] = key;
      a.missed_indices[at] = (int32_t)i;
    }
  }
  if (MODE != kLookupValues) return;

  /* copy stage: 64 rows x units-per-row spread over the 64 lanes.  All loads
   * of a batch are issued before the first store, so a wavefront keeps up to
   * kBatch KB of value rows in flight (the whole 16 KB for 256-byte rows). */
  using T = typename VecType<VEC>::type;
  const uint32_t units = v.value_bytes / VEC;
  const uint32_t total = units * kWave;
  const bool pow2 = (units & (units - 1)) == 0;
  const uint32_t sh = 31 - __clz(units);
  if constexpr (VEC == 16) {
    /* Rows of 16 to 1024 bytes whose size is a power of two, all in HBM, slot numbers below
     * 2^32 (every decision here is the same for the whole wavefront): lane L then always
     * moves unit L mod units of a row, and in pass b the row of key (L / units) + b * (64 /
     * units), so the slot numbers are read from LDS in one go and an address costs one
     * multiply-add.  The general form below spends more instructions on addresses than
     * the memory system needs time for the rows. */
    if (pow2 && units <= kWave && v.hbm_slots >= v.capacity && v.capacity <= 0xFFFFFFFFull) {
      constexpr int kB = 16;
      const uint32_t c = lane & (units - 1);
      const uint32_t kk0 = lane >> sh;
      const uint32_t kstep = kWave >> sh;
      const uint8_t* const src0 = v.values + c * 16;
      uint8_t* const dst0 = a.out_values + (base + kk0) * v.value_bytes + c * 16;
      const uint64_t dstep = (uint64_t)kstep * v.value_bytes;
      /* with all 64 keys found nothing below is conditional, and the stores start as the
       * first rows arrive instead of after the last one */
      const bool all = __ballot(my_slot >= 0) == ~0ull;
      auto move = [&](auto all_found) {
        constexpr bool ALL = decltype(all_found)::value;
        for (uint32_t b0 = 0; b0 < units; b0 += kB) {
          int64_t sl[kB];
          u32x4_t buf[kB];
          if (ALL && units >= kB) {
#pragma unroll
            for (int b = 0; b < kB; b++) sl[b] = s_slot[kk0 + (b0 + b) * kstep];
#pragma unroll
            for (int b = 0; b < kB; b++)
              buf[b] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(
                  src0 + (uint64_t)(uint32_t)sl[b] * v.value_bytes));
#pragma unroll
            for (int b = 0; b < kB; b++)
              __builtin_nontemporal_store(buf[b],
                                          reinterpret_cast<u32x4_t*>(dst0 + (b0 + b) * dstep));
          } else {
#pragma unroll
            for (int b = 0; b < kB; b++)
              sl[b] = b0 + b < units ? s_slot[kk0 + (b0 + b) * kstep] : -1;
#pragma unroll
            for (int b = 0; b < kB; b++)
              if (sl[b] >= 0)
                buf[b] = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(
                    src0 + (uint64_t)(uint32_t)sl[b] * v.value_bytes));
#pragma unroll
            for (int b = 0; b < kB; b++)
              if (sl[b] >= 0)
                __builtin_nontemporal_store(buf[b],
                                            reinterpret_cast<u32x4_t*>(dst0 + (b0 + b) * dstep));
          }
        }
      };
      if (all)
        move(std::true_type{});
      else
        move(std::false_type{});
      return;
    }
  }
  constexpr int kBatch = VEC == 16 ? 16 : 4;
  for (uint32_t idx0 = lane; idx0 < total; idx0 += kWave * kBatch) {
    T buf[kBatch];
#pragma unroll
    for (int b = 0; b < kBatch; b++) {
      const uint32_t idx = idx0 + b * kWave;
      buf[b] = T{};
      if (idx < total) {
        const uint32_t kk = pow2 ? (idx >> sh) : (idx / units);
        const uint32_t c = idx - kk * units;
        const int64_t slot = s_slot[kk];
        if (slot >= 0) {
          const T* src = reinterpret_cast<const T*>(value_row(v, (uint64_t)slot)) + c;
          if constexpr (VEC == 16) {
            /* a row is read once: streaming (non-temporal) loads, measured ~6 %
             * faster here than plain ones */
            const u32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(src));
            buf[b] = make_uint4(t.x, t.y, t.z, t.w);
          } else {
            buf[b] = *src;
          }
        }
      }
    }
#pragma unroll
    for (int b = 0; b < kBatch; b++) {
      const uint32_t idx = idx0 + b * kWave;
      if (idx < total) {
        const uint32_t kk = pow2 ? (idx >> sh) : (idx / units);
        const uint32_t c = idx - kk * units;
        if (s_slot[kk] >= 0) {
          T* dst = reinterpret_cast<T*>(a.out_values + (base + kk) * v.value_bytes) + c;
          if constexpr (VEC == 16) {
            /* streaming store: the output is not read again here, and rows left dirty
             * in the caches would be written back at the expense of the next call
             * (measured: find itself 2 % slower, a following upsert 6 % faster) */
            const u32x4_t t = {buf[b].x, buf[b].y, buf[b].z, buf[b].w};
            __builtin_nontemporal_store(t, reinterpret_cast<u32x4_t*>(dst));
          } else {
            *dst = buf[b];
          }
        }
      }
    }
  }
}

}  // namespace hkv
#endif
