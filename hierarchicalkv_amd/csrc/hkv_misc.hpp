/*
 * Table maintenance kernels: initial fill, clear, erase, size, and the
 * built-in export predicates.
 */
#ifndef HKV_MISC_HPP_
#define HKV_MISC_HPP_

#include "hkv_lookup.hpp"

namespace hkv {

/* initialize_buckets (core_kernels.cuh:169-292) and clear_kernel (:656-676) in
 * one grid-wide fill: key = EMPTY, digest = EMPTY marker, size = 0, score bounds = 0; scores
 * are zeroed only at creation (clear leaves scores and values as they are).
 * One thread per 16 slots. */
__global__ void __launch_bounds__(256)
fill_kernel(View v, int zero_scores) {
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t groups = v.capacity / 16;
  if (t < groups) {
    const uint32_t e4 = v.empty_digest * 0x01010101u;
    reinterpret_cast<uint4*>(v.digests)[t] = make_uint4(e4, e4, e4, e4);
    uint64_t* k = v.keys + t * 16;
#pragma unroll
    for (int q = 0; q < 16; q++) k[q] = v.empty_key;
    if (zero_scores) {
      uint64_t* s = v.scores + t * 16;
#pragma unroll
      for (int q = 0; q < 16; q++) s[q] = 0;
    }
    if (v.bounds) v.bounds[t] = 0; /* one per 16 slots */
  }
  if (v.sizes && t < v.buckets_num) v.sizes[t] = 0;
}

/* one sample of the constant-rate device counter (table creation: see Clock) */
__global__ void clock_sample_kernel(unsigned long long* out) { *out = wall_clock64(); }

/* remove_kernel (core_kernels.cuh:679-741): free the slot.
 * EXCLUSIVE: the call is the only one on the table while it runs (it holds the inserter role
 * of the group lock), so the key word is overwritten with a plain store as in the reference
 * (core_kernels.cuh:723-737; like there, a batch that names a key twice in different
 * wavefronts may count it twice).  Otherwise the slot changes hands with a compare-and-swap.
 * A key that an 8-lane tile holds twice is erased once.  No counter is kept per bucket (the
 * number of keys of a table is the number of digests that are not the EMPTY marker, counted
 * when somebody asks), so an erase is two stores. */
template <bool EXCLUSIVE>
__global__ void __launch_bounds__(kWave)
erase_kernel(View v, const uint64_t* keys, uint64_t n) {
  __shared__ KeyMeta s_meta[kWave];
  __shared__ int64_t s_slot[kWave];
  const int lane = threadIdx.x;
  const uint64_t i = (uint64_t)blockIdx.x * kWave + lane;
  const uint64_t key = stage_keys(v, keys, n, i, s_meta, s_slot, lane);
  __syncthreads();
  probe_wave<false, false>(v, s_meta, s_slot, nullptr, nullptr, lane);
  __syncthreads();
  const int64_t slot = s_slot[lane];
  const int tile_base = lane & ~(kTile - 1), j = lane & (kTile - 1);
  bool mine = slot >= 0;
#pragma unroll
  for (int q = 0; q < kTile; q++) {
    const int64_t other = __shfl((long long)slot, tile_base + q);
    if (q < j && other == slot) mine = false; /* the same key earlier in the tile */
  }
  bool erased = false;
  if (mine) {
    /* The slot becomes a free slot outright: EMPTY key, EMPTY digest.  The reference leaves a
     * tombstone (RECLAIM key, score 0, core_kernels.cuh:723-737) because its probes stop at the
     * first EMPTY key; here every probe looks at all 128 digests, a free slot in the middle of a
     * bucket hides nothing, and the next insert takes it through the free-slot path instead of
     * finding it as the bucket's lowest score.  Which slot a key lands in shows in no result;
     * one store and one score write less per key. */
    if (EXCLUSIVE) {
      erased = true;
      v.keys[slot] = v.empty_key;
    } else {
      uint64_t seen = key;
      erased = cas_lock(v.keys + slot, seen, v.locked_key);
    }
    if (EXCLUSIVE && erased) v.digests[slot] = v.empty_digest;
  }
  if (!EXCLUSIVE) {
    /* Without the group lock an inserter of another launch may be looking: the digest goes out
     * as a store that every compute die sees, it is complete before the key word opens, and
     * the key word opens last.  (A digest store that came later than the key word would land
     * on the digest of the key that took the slot in between.) */
    if (erased) st_u8(v.digests + slot, (uint8_t)v.empty_digest);
    wait_stores();
    if (erased) st_u64(v.keys + slot, v.empty_key);
  }
}

/* Number of keys of the table (the reference sums per-bucket counters, SumOp over buckets_size,
 * core_kernels.cuh:1395-1423).  A slot holds a key exactly when its digest is not the EMPTY
 * marker (a live key never stores that byte, erase and clear put it back), so the count is one
 * streaming pass over the digest array, 16 bytes per lane and step; no call that inserts or
 * erases pays for a counter.  The first `buckets` buckets are counted (all of them for size(),
 * the first 1024 for the load-factor estimate, merlin_hashtable.cuh:3796-3830).
 * Few blocks: the one word they all add to takes one update at a time. */
__global__ void __launch_bounds__(256)
size_kernel(View v, uint64_t buckets, unsigned long long* out) {
  uint64_t local = 0;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  const uint64_t tid = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t groups = buckets * (kBucketSize / 16);
  const uint32_t e4 = v.empty_digest * 0x01010101u;
  const uint4* d = reinterpret_cast<const uint4*>(v.digests);
  /* four loads in flight per lane */
  uint64_t g = tid;
  for (; g + 3 * stride < groups; g += 4 * stride) {
    const uint4 x0 = d[g], x1 = d[g + stride], x2 = d[g + 2 * stride], x3 = d[g + 3 * stride];
    local += 64 - __popc(match16(x0, e4)) - __popc(match16(x1, e4)) - __popc(match16(x2, e4)) -
             __popc(match16(x3, e4));
  }
  for (; g < groups; g += stride) local += 16 - __popc(match16(d[g], e4));
  __shared__ unsigned long long s_part[4];
  for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = local;
  __syncthreads();
  if (threadIdx.x == 0) {
    const unsigned long long total = s_part[0] + s_part[1] + s_part[2] + s_part[3];
    if (total) atomicAdd(out, total);
  }
}

/*
 * Rehash into a table with twice the buckets (rehash_kernel_for_fast_mode,
 * core_kernels.cuh:540-591).  With g = hash modulo capacity and the bucket
 * count doubling from B to 2B, a key of bucket b lands in bucket b or b + B
 * of the new table, and both start out empty: every entry can keep its slot
 * position, so no destination search and no compaction is needed (positions
 * are not observable through the API).  Tombstones stay in bucket b.  One
 * wavefront per 64 slots; it moves the rows of its live keys together.
 */
__global__ void __launch_bounds__(256)
rehash_kernel(View src, View dst) {
  const int lane = lane_id();
  const uint64_t wave = ((uint64_t)blockIdx.x * blockDim.x + threadIdx.x) / kWave;
  const uint64_t s = wave * kWave + lane;
  if (wave * kWave >= src.capacity) return;
  const uint64_t b = s >> 7;
  const uint32_t p = (uint32_t)(s & 127u);
  const uint64_t key = src.keys[s];
  const bool tomb = key == src.reclaim_key;
  const bool live = key != src.empty_key && !tomb;
  uint64_t nb = b;
  if (live) {
    uint32_t bkt, start, digest;
    locate(dst, key, bkt, start, digest);
    nb = bkt;
  }
  const uint64_t d = nb * kBucketSize + p;
  if (live || tomb) {
    dst.keys[d] = key;
    dst.digests[d] = src.digests[s];
    dst.scores[d] = src.scores[s];
  }
  unsigned long long rest = __ballot(live);
  while (rest) {
    const int l = __ffsll(rest) - 1;
    rest &= rest - 1;
    const uint64_t dl = __shfl((unsigned long long)d, l);
    wave_copy_row(value_row(dst, dl), value_row(src, wave * kWave + l), src.value_bytes, lane);
  }
}

/* keys in the first n buckets (fast_load_factor, merlin_hashtable.cuh:3796-3830); one workgroup,
 * which stores its whole result in one write */
__global__ void __launch_bounds__(256)
load_sample_kernel(View v, uint32_t n, unsigned long long* out) {
  __shared__ unsigned long long s_part[4];
  unsigned long long local = 0;
  const uint32_t e4 = v.empty_digest * 0x01010101u;
  const uint4* d = reinterpret_cast<const uint4*>(v.digests);
  for (uint32_t g = threadIdx.x; g < n * (kBucketSize / 16); g += 256) local += 16 - __popc(match16(d[g], e4));
  for (int off = 32; off > 0; off >>= 1) local += __shfl_xor(local, off);
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = local;
  __syncthreads();
  if (threadIdx.x == 0) *out = s_part[0] + s_part[1] + s_part[2] + s_part[3];
}

__global__ void zero_u64_kernel(unsigned long long* p) { *p = 0; }
/* the table's count of LOCKED slots, all its words (one thread each) */
__global__ void zero_locked_kernel(unsigned long long* count) { count[threadIdx.x * kLockedStride] = 0; }
__global__ void zero_i32_kernel(int32_t* p) { *p = 0; }
/* n 32-bit words from p on become zero (n a multiple of 4, p aligned to 16 bytes) */
__global__ void __launch_bounds__(256)
zero_words_kernel(uint32_t* p, uint64_t n) {
  const uint64_t q = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (q * 4 < n) reinterpret_cast<uint4*>(p)[q] = make_uint4(0, 0, 0, 0);
}

/* What the score bounds are rebuilt against and where the limits of the next upsert live. */
struct BoundsRebuild {
  Clock clock;
  int32_t strategy;
  uint64_t epoch;
  unsigned long long* clock_word;       /* hardware clock: gets a reading, which the upsert that
                                           follows takes as its own limit (UpsertArgs::bound_cap_in) */
  const unsigned long long* floor_word; /* scores from the caller: the lowest score of the batch
                                           that is about to run (score_floor_kernel) */
  unsigned long long* ceil_word;        /* with floor_word: gets the limit the bounds were made with */
};

/* The score bounds from scratch: for every line of 16 slots the lowest score of its keys, but
 * nothing above a value that no score written from now on is below (as UpsertArgs::bound_cap),
 * and 0 for a line without keys.  A free slot does not count: what it gets later is a score of
 * that time.  Eight lanes per line, one wavefront per 8 lines; the caller has the table to
 * itself. */
__global__ void __launch_bounds__(256)
rebuild_bounds_kernel(View v, BoundsRebuild r) {
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (t == 0 && r.clock_word) *r.clock_word = now_ns(r.clock, 0);
  /* deterministic clock: the base of the call that is about to run; hardware clock: now, which
   * is before anything that call writes; scores from the caller: the lowest of that call */
  uint64_t cap = r.clock.mode == 1 ? r.clock.base : now_ns(r.clock, 0);
  if (r.strategy == HKV_EPOCH_LRU) cap = (r.epoch << 32) | ((cap >> 20) & kLow32);
  if (r.floor_word) cap = *r.floor_word;
  if (t == 0 && r.ceil_word) *r.ceil_word = cap;
  const uint64_t line = t >> 3;
  const int j = (int)(t & 7);
  if (line >= v.capacity / 16) return; /* whole tiles leave together: lines are a multiple of 8 */
  const uint4 k = *reinterpret_cast<const uint4*>(v.keys + line * 16 + j * 2);
  const uint4 s = *reinterpret_cast<const uint4*>(v.scores + line * 16 + j * 2);
  const uint64_t k0 = k.x | ((uint64_t)k.y << 32), k1 = k.z | ((uint64_t)k.w << 32);
  const uint64_t s0 = s.x | ((uint64_t)s.y << 32), s1 = s.z | ((uint64_t)s.w << 32);
  /* a tombstone holds score 0 and is what a search should find first; LOCKED slots (lock_keys)
   * hold a key with its score */
  uint64_t m = kMaxScore;
  if (k0 != v.empty_key) m = s0;
  if (k1 != v.empty_key && s1 < m) m = s1;
  m = tile_min(m);
  if (j == 0) v.bounds[line] = m == kMaxScore ? 0 : (m < cap ? m : cap);
}

/* The lowest score a batch can leave in the table, for the strategies that take scores from the
 * caller: Customized and LFU store the caller's score for a new key (an LFU key that is found
 * ends above it), EpochLFU the epoch over its low half (kernel_utils.cuh:332-371, 464-517,
 * 567-593).  `out` must hold kMaxScore when the kernel starts: `next`, the word the following
 * call will use, is reset here, and the two words are used in turn.  Few, large workgroups:
 * updates of one word are served one at a time. */
__global__ void __launch_bounds__(1024)
score_floor_kernel(const uint64_t* scores, uint64_t n, int strategy, uint64_t epoch,
                   unsigned long long* out, unsigned long long* next) {
  __shared__ unsigned long long s_part[16];
  uint64_t m = kMaxScore;
  const uint64_t stride = (uint64_t)gridDim.x * blockDim.x;
  for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
    uint64_t x = scores[i];
    if (strategy == HKV_EPOCH_LFU && epoch != kIgnoredEpoch) x = (epoch << 32) | (x & kLow32);
    m = x < m ? x : m;
  }
  for (int off = 32; off > 0; off >>= 1) {
    const uint64_t o = __shfl_xor((unsigned long long)m, off);
    m = o < m ? o : m;
  }
  if ((threadIdx.x & 63) == 0) s_part[threadIdx.x >> 6] = m;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < (int)(blockDim.x >> 6); w++) m = s_part[w] < m ? s_part[w] : m;
    __hip_atomic_fetch_min(out, (unsigned long long)m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (blockIdx.x == 0) *next = kMaxScore;
  }
}

/* ---- built-in predicates (hkv_predicate) -------------------------------------- */

struct PredAlways {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t&,
                                             const uint64_t&, const uint64_t&) const {
    return true;
  }
};
struct PredScoreLt {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s < th;
  }
};
struct PredScoreLe {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s <= th;
  }
};
struct PredScoreGt {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s > th;
  }
};
struct PredScoreGe {
  __device__ __forceinline__ bool operator()(const uint64_t&, uint64_t& s,
                                             const uint64_t&, const uint64_t& th) const {
    return s >= th;
  }
};
struct PredKeyHigh16AndScoreLt {
  __device__ __forceinline__ bool operator()(const uint64_t& k, uint64_t& s,
                                             const uint64_t& pat,
                                             const uint64_t& th) const {
    return (k & UINT64_C(0xFFFF000000000000)) == pat && s < th;
  }
};

}  // namespace hkv
#endif
