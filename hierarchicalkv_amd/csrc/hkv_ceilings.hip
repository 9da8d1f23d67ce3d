/*
 * Memory-system ceilings for the table kernels: kernels that issue the access pattern of
 * find and of insert_or_assign at a given table shape with no table logic in them (no
 * hashing of real keys, no comparisons, no dependent loads: every address is a function of
 * the thread index and a salt; one variant of find's pattern chains its four groups of loads
 * as the real kernel has to), plus the plain streaming, gather, scatter and small-access
 * rates the patterns are made of.  What such a kernel takes is what the memory system
 * needs for the bytes alone; the distance of a real kernel from it is what its logic and its
 * dependent round trips cost.
 *
 * Measurement tool, built as its own library (libhkv_ceilings.so) and loaded by
 * bench.py --ceilings only; nothing in libhkv.so depends on it.  It owns its buffers
 * (hipMalloc at first use, sized like a table of the requested shape).
 */
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint64_t mix(uint64_t k) {
  k ^= k >> 33;
  k *= 0xff51afd7ed558ccdULL;
  k ^= k >> 33;
  k *= 0xc4ceb9fe1a85ec53ULL;
  k ^= k >> 33;
  return k;
}

/* store / load flavours used by the table kernels */
__device__ __forceinline__ void st16_wt(void* p, u32x4 x) { /* write-through, non-temporal */
  asm volatile("global_store_dwordx4 %0, %1, off sc1 nt\n\ts_nop 1" : : "v"(p), "v"(x) : "memory");
}
__device__ __forceinline__ void st16_nt(u32x4* p, u32x4 x) { __builtin_nontemporal_store(x, p); }
__device__ __forceinline__ u32x4 ld16_nt(const u32x4* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ void st8_wt(uint64_t* p, uint64_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ void st1_wt(uint8_t* p, uint8_t x) {
  __hip_atomic_store(p, x, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct Shape {
  uint64_t buckets;   /* power of two */
  uint32_t row_bytes; /* multiple of 16 */
  uint64_t n;         /* keys per launch */
};

struct Buffers {
  uint8_t* digests;  /* buckets * 128 */
  uint64_t* keys;    /* buckets * 128 */
  uint64_t* scores;  /* buckets * 128 */
  uint8_t* rows;     /* buckets * 128 * row_bytes */
  uint8_t* in_rows;  /* n * row_bytes */
  uint8_t* out_rows; /* n * row_bytes */
  uint64_t* in_keys; /* n */
  uint8_t* flags;    /* n */
  uint32_t* small;   /* buckets words: a 4-byte-per-bucket side array */
  uint32_t* sink;
};

/* ---- streaming ---------------------------------------------------------------------------- */

__global__ void k_stream_read(const u32x4* p, uint64_t units, uint32_t* sink) {
  uint32_t acc = 0;
  for (uint64_t u = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; u < units;
       u += (uint64_t)gridDim.x * blockDim.x) {
    const u32x4 x = ld16_nt(p + u);
    acc += x.x ^ x.w;
  }
  if (acc == 0x12345u) *sink = acc;
}
__global__ void k_stream_write(u32x4* p, uint64_t units) {
  for (uint64_t u = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; u < units;
       u += (uint64_t)gridDim.x * blockDim.x) {
    const u32x4 x = {(uint32_t)u, 1, 2, 3};
    st16_nt(p + u, x);
  }
}
__global__ void k_stream_copy(const u32x4* s, u32x4* d, uint64_t units) {
  for (uint64_t u = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; u < units;
       u += (uint64_t)gridDim.x * blockDim.x)
    st16_nt(d + u, ld16_nt(s + u));
}

/* ---- rows: random rows of the table <-> a dense array, 16 bytes per lane ------------------------ */

__global__ void k_row_gather(Shape sh, Buffers b, uint64_t salt) {
  const uint32_t upr = sh.row_bytes / 16;
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t r = t / upr;
  if (r >= sh.n) return;
  const uint64_t row = mix(r + salt) & (sh.buckets * 128 - 1);
  const u32x4* src = reinterpret_cast<const u32x4*>(b.rows + row * sh.row_bytes) + (t - r * upr);
  st16_nt(reinterpret_cast<u32x4*>(b.out_rows) + t, ld16_nt(src));
}
__global__ void k_row_scatter(Shape sh, Buffers b, uint64_t salt) {
  const uint32_t upr = sh.row_bytes / 16;
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t r = t / upr;
  if (r >= sh.n) return;
  const uint64_t row = mix(r + salt) & (sh.buckets * 128 - 1);
  u32x4* dst = reinterpret_cast<u32x4*>(b.rows + row * sh.row_bytes) + (t - r * upr);
  st16_wt(dst, ld16_nt(reinterpret_cast<const u32x4*>(b.in_rows) + t));
}

/* ---- the access pattern of find ------------------------------------------------------------------
 * One wavefront per 64 keys.  Per key: the 8-byte key of the batch, the bucket's 128-byte
 * digest line (8 lanes x 16 bytes), one 8-byte key word of the table (a whole line of
 * traffic), a second one for `extra_pm` keys in 1000 (false digest matches), the row (row_bytes)
 * gathered and written to the dense output, one found flag. */
/* zero, but only known once `x` has arrived: makes an address depend on a load */
__device__ __forceinline__ uint32_t zero_after(uint32_t x) {
  uint32_t z;
  asm volatile("v_and_b32 %0, 0, %1" : "=v"(z) : "v"(x));
  return z;
}

/* CHAIN: the same accesses, but each group of addresses is only known when the group before
 * it has arrived, as in the real kernel (key of the batch -> digest line -> key word of the
 * table -> row): four round trips in a row instead of one. */
template <bool CHAIN>
__global__ void __launch_bounds__(64)
k_find_pattern(Shape sh, Buffers b, uint64_t salt, uint32_t extra_pm) {
  const int lane = threadIdx.x, tile = lane >> 3, j = lane & 7;
  const uint64_t base = (uint64_t)blockIdx.x * 64;
  uint64_t acc = b.in_keys[base + lane];
  if (CHAIN) salt += zero_after((uint32_t)acc);
  /* digest lines: tile t reads the lines of keys 8t..8t+7 */
  uint4 dg[8];
#pragma unroll
  for (int r = 0; r < 8; r++) {
    const uint64_t bk = mix(base + tile * 8 + r + salt) & (sh.buckets - 1);
    dg[r] = *reinterpret_cast<const uint4*>(b.digests + bk * 128 + j * 16);
  }
#pragma unroll
  for (int r = 0; r < 8; r++) acc += dg[r].x ^ dg[r].w;
  if (CHAIN) salt += zero_after((uint32_t)acc);
  /* key words: lane L verifies key L */
  {
    const uint64_t h = mix(base + lane + salt);
    const uint64_t bk = h & (sh.buckets - 1);
    const uint32_t p = (uint32_t)(h >> 40) & 127u;
    acc += b.keys[bk * 128 + p];
    if ((uint32_t)((h >> 48) % 1000) < extra_pm) acc += b.keys[bk * 128 + ((p + 64) & 127u)];
  }
  if (acc == 0x123456789ULL) *b.sink = 1;
  b.flags[base + lane] = 1;
  if (CHAIN) salt += zero_after((uint32_t)acc);
  /* rows: 64 rows x units spread over the 64 lanes, loads before stores */
  const uint32_t upr = sh.row_bytes / 16;
  const uint32_t total = upr * 64;
  for (uint32_t idx0 = lane; idx0 < total; idx0 += 64 * 16) {
    u32x4 buf[16];
#pragma unroll
    for (int q = 0; q < 16; q++) {
      const uint32_t idx = idx0 + q * 64;
      buf[q] = u32x4{0, 0, 0, 0};
      if (idx < total) {
        const uint32_t kk = idx / upr, c = idx - kk * upr;
        const uint64_t h = mix(base + kk + salt);
        const uint64_t slot = (h & (sh.buckets - 1)) * 128 + ((uint32_t)(h >> 40) & 127u);
        buf[q] = ld16_nt(reinterpret_cast<const u32x4*>(b.rows + slot * sh.row_bytes) + c);
      }
    }
#pragma unroll
    for (int q = 0; q < 16; q++) {
      const uint32_t idx = idx0 + q * 64;
      if (idx < total)
        st16_nt(reinterpret_cast<u32x4*>(b.out_rows + base * sh.row_bytes) + idx, buf[q]);
    }
  }
}

/* ---- the access pattern of insert_or_assign into a full table ---------------------------------------
 * As find's pattern for the probe (key, digest line, key word(s)); then
 *   even keys ("present"): the row written from the dense input, one 8-byte score store;
 *   odd keys ("absent"):   the bucket's 128 scores read (1 KB, 8 lanes x 8 lines), the row
 *                          written, 8-byte key and score stores and a 1-byte digest store.
 * `locks` adds what the slot-lock protocol spends: a compare-and-swap and an unlock store per
 * present key, an exchange and a score re-read per absent key (the key store of an absent
 * key doubles as its unlock).
 * locks == 3: a table with free slots.  An absent key reads no scores: it takes a free slot with
 * a compare-and-swap; a quarter of the absent keys fetch a key line for a false digest match. */
template <bool CHAIN>
__global__ void __launch_bounds__(64)
k_upsert_pattern(Shape sh, Buffers b, uint64_t salt, uint32_t extra_pm, int locks) {
  const int lane = threadIdx.x, tile = lane >> 3, j = lane & 7;
  const uint64_t base = (uint64_t)blockIdx.x * 64;
  uint64_t acc = b.in_keys[base + lane];
  /* CHAIN: as in k_find_pattern, every group of addresses waits for the group before it:
   * batch key -> digest line -> key word (and compare-and-swap) -> score scan -> exchange
   * and score re-read -> stores -> unlock */
  if (CHAIN) salt += zero_after((uint32_t)acc);
  uint4 dg[8];
#pragma unroll
  for (int r = 0; r < 8; r++) {
    const uint64_t bk = mix(base + tile * 8 + r + salt) & (sh.buckets - 1);
    dg[r] = *reinterpret_cast<const uint4*>(b.digests + bk * 128 + j * 16);
  }
#pragma unroll
  for (int r = 0; r < 8; r++) acc += dg[r].x ^ dg[r].w;
  if (CHAIN) salt += zero_after((uint32_t)acc);
  const uint64_t h = mix(base + lane + salt);
  const uint64_t bk = h & (sh.buckets - 1);
  const uint32_t p = (uint32_t)(h >> 40) & 127u;
  uint64_t slot = bk * 128 + p;
  const bool absent = lane & 1;
  const bool free_mode = locks == 3;
  if (!(free_mode && absent) || (uint32_t)((h >> 52) % 1000) < 250u) acc += b.keys[slot];
  if ((uint32_t)((h >> 48) % 1000) < extra_pm) acc += b.keys[bk * 128 + ((p + 64) & 127u)];
  if (locks) {
    if (!absent || free_mode) {
      uint64_t expect = acc;
      __hip_atomic_compare_exchange_strong(b.keys + slot, &expect, acc, __ATOMIC_RELAXED,
                                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      acc += expect;
    }
  }
  if (CHAIN) salt += zero_after((uint32_t)acc);
  /* score scans of the absent keys: keys 8t+1, 8t+3, 8t+5, 8t+7 of each tile, two in flight;
   * with score bounds (locks == 2): the bucket's 8 bounds (64 bytes), then one score line */
  if (free_mode) {
    /* no victim search */
  } else if (locks == 2) {
    uint64_t bd[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
      const uint64_t bk2 = mix(base + tile * 8 + 2 * w + 1 + salt) & (sh.buckets - 1);
      bd[w] = reinterpret_cast<const uint64_t*>(b.digests)[bk2 * 8 + j];
    }
#pragma unroll
    for (int w = 0; w < 4; w++) acc += bd[w];
    if (CHAIN) salt += zero_after((uint32_t)acc);
    uint4 ln[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
      const uint64_t h2 = mix(base + tile * 8 + 2 * w + 1 + salt);
      const uint64_t bk2 = h2 & (sh.buckets - 1);
      ln[w] = *reinterpret_cast<const uint4*>(b.scores + bk2 * 128 + ((h2 >> 40) & 7) * 16 + j * 2);
    }
#pragma unroll
    for (int w = 0; w < 4; w++) acc += ln[w].x ^ ln[w].z;
  } else
#pragma unroll
  for (int r = 1; r < 8; r += 4) {
    uint4 sc[2][8];
#pragma unroll
    for (int w = 0; w < 2; w++) {
      const uint64_t bk2 = mix(base + tile * 8 + r + 2 * w + salt) & (sh.buckets - 1);
#pragma unroll
      for (int it = 0; it < 8; it++)
        sc[w][it] = *reinterpret_cast<const uint4*>(b.scores + bk2 * 128 + it * 16 + j * 2);
    }
#pragma unroll
    for (int w = 0; w < 2; w++)
#pragma unroll
      for (int it = 0; it < 8; it++) acc += sc[w][it].x ^ sc[w][it].z;
  }
  if (CHAIN) slot += zero_after((uint32_t)acc);
  if (locks && absent && !free_mode) {
    acc += __hip_atomic_exchange(b.keys + slot, acc, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    if (CHAIN) slot += zero_after((uint32_t)acc);
    acc += __hip_atomic_load(b.scores + slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  if (CHAIN) {
    const uint32_t z = zero_after((uint32_t)acc);
    slot += z;
    salt += z;
  }
  if (acc == 0x123456789ULL) *b.sink = 1;
  /* metadata stores */
  st8_wt(b.scores + slot, acc);
  if (absent) {
    st1_wt(b.digests + slot, (uint8_t)acc);
    st8_wt(b.keys + slot, acc);
    if (locks == 2) st8_wt(reinterpret_cast<uint64_t*>(b.digests) + (slot >> 4), acc);
  }
  /* rows: dense input -> table rows, 64 rows x units over the 64 lanes */
  const uint32_t upr = sh.row_bytes / 16;
  const uint32_t total = upr * 64;
  for (uint32_t idx0 = lane; idx0 < total; idx0 += 64 * 16) {
    u32x4 buf[16];
#pragma unroll
    for (int q = 0; q < 16; q++) {
      const uint32_t idx = idx0 + q * 64;
      buf[q] = u32x4{0, 0, 0, 0};
      if (idx < total)
        buf[q] = ld16_nt(reinterpret_cast<const u32x4*>(b.in_rows + base * sh.row_bytes) + idx);
    }
#pragma unroll
    for (int q = 0; q < 16; q++) {
      const uint32_t idx = idx0 + q * 64;
      if (idx < total) {
        const uint32_t kk = idx / upr, c = idx - kk * upr;
        const uint64_t h2 = mix(base + kk + salt);
        const uint64_t s2 = (h2 & (sh.buckets - 1)) * 128 + ((uint32_t)(h2 >> 40) & 127u);
        st16_wt(b.rows + s2 * sh.row_bytes + c * 16, buf[q]);
      }
    }
  }
  if (locks && !absent) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    st8_wt(b.keys + slot, acc);
  }
}

/* ---- the access pattern of the calls that move no rows -------------------------------------------------
 * Probe as find's (batch key, digest line, one key word, a second one for `extra_pm` keys in 1000);
 * kind 0 (find* / contains): one 8-byte result and one flag per key;
 * kind 1 (erase with the table to itself): an 8-byte key store and a 1-byte digest store into the
 *        table. */
__global__ void __launch_bounds__(64)
k_norow_pattern(Shape sh, Buffers b, uint64_t salt, uint32_t extra_pm, int kind) {
  const int lane = threadIdx.x, tile = lane >> 3, j = lane & 7;
  const uint64_t base = (uint64_t)blockIdx.x * 64;
  uint64_t acc = b.in_keys[base + lane];
  salt += zero_after((uint32_t)acc);
  uint4 dg[8];
#pragma unroll
  for (int r = 0; r < 8; r++) {
    const uint64_t bk = mix(base + tile * 8 + r + salt) & (sh.buckets - 1);
    dg[r] = *reinterpret_cast<const uint4*>(b.digests + bk * 128 + j * 16);
  }
#pragma unroll
  for (int r = 0; r < 8; r++) acc += dg[r].x ^ dg[r].w;
  salt += zero_after((uint32_t)acc);
  const uint64_t h = mix(base + lane + salt);
  const uint64_t bk = h & (sh.buckets - 1);
  const uint32_t p = (uint32_t)(h >> 40) & 127u;
  uint64_t slot = bk * 128 + p;
  acc += b.keys[slot];
  if ((uint32_t)((h >> 48) % 1000) < extra_pm) acc += b.keys[bk * 128 + ((p + 64) & 127u)];
  slot += zero_after((uint32_t)acc);
  if (acc == 0x123456789ULL) *b.sink = 1;
  if (kind == 0) {
    reinterpret_cast<uint64_t*>(b.out_rows)[base + lane] = acc;
    b.flags[base + lane] = 1;
  } else {
    b.keys[slot] = acc;
    b.digests[slot] = (uint8_t)acc;
  }
}

/* ---- small accesses: n operations, one per random 128-byte line of a region -------------------------
 * kind 0: 8-byte store   1: 1-byte store   2: 8-byte load   3: 64-bit compare-and-swap
 *      4: 64-bit exchange   5: 64-byte aligned chunk written by 4 lanes   6: 16-byte store
 *      7: 32-bit exchange on the 4-byte-per-bucket side array (a region of buckets * 4 bytes) */
__global__ void k_small(Shape sh, Buffers b, uint64_t n, uint64_t salt, int kind) {
  const uint64_t t = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const uint64_t lines = sh.buckets * 8; /* 128-byte lines of the scores array */
  if (kind == 5) {
    const uint64_t r = t >> 2;
    if (r >= n) return;
    const uint64_t line = mix(r + salt) & (lines - 1);
    const u32x4 x = {(uint32_t)t, 1, 2, 3};
    st16_wt(reinterpret_cast<uint8_t*>(b.scores) + line * 128 + (t & 3) * 16, x);
    return;
  }
  if (t >= n) return;
  const uint64_t line = mix(t + salt) & (lines - 1);
  uint64_t* w = b.scores + line * 16 + (t & 15);
  uint64_t acc = 0;
  switch (kind) {
    case 0: st8_wt(w, t); break;
    case 1: st1_wt(reinterpret_cast<uint8_t*>(w), (uint8_t)t); break;
    case 2: acc = __hip_atomic_load(w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break;
    case 3: {
      uint64_t e = t;
      __hip_atomic_compare_exchange_strong(w, &e, t + 1, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
      acc = e;
      break;
    }
    case 4: acc = __hip_atomic_exchange(w, t, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break;
    case 6: {
      const u32x4 x = {(uint32_t)t, 1, 2, 3};
      st16_wt(reinterpret_cast<uint8_t*>(b.scores) + line * 128 + (t & 7) * 16, x);
      break;
    }
    default:
      acc = __hip_atomic_exchange(b.small + (mix(t + salt) & (sh.buckets - 1)), (uint32_t)t,
                                  __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      break;
  }
  if (acc == 0x123456789ULL) *b.sink = 1;
}

Shape g_shape{};
Buffers g_buf{};
bool g_ready = false;
char g_err[256];

#define CK(expr)                                                                        \
  do {                                                                                  \
    hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess) {                                                             \
      snprintf(g_err, sizeof g_err, "%s:%d %s: %s", __FILE__, __LINE__, #expr,          \
               hipGetErrorString(e_));                                                  \
      return 1;                                                                         \
    }                                                                                   \
  } while (0)

void release() {
  void* all[] = {g_buf.digests, g_buf.keys,    g_buf.scores, g_buf.rows,  g_buf.in_rows,
                 g_buf.out_rows, g_buf.in_keys, g_buf.flags,  g_buf.small, g_buf.sink};
  for (void* p : all)
    if (p) (void)hipFree(p);
  g_buf = Buffers{};
  g_ready = false;
}

}  // namespace

extern "C" {

const char* hkv_ceilings_last_error(void) { return g_err; }

/* Buffers for a table of `buckets` (a power of two) buckets with rows of `row_bytes`, and a
 * batch of `n` keys (a multiple of 64). */
int hkv_ceilings_setup(uint64_t buckets, uint32_t row_bytes, uint64_t n) {
  if (buckets == 0 || (buckets & (buckets - 1)) || row_bytes == 0 || (row_bytes & 15) || n == 0 ||
      (n & 63)) {
    snprintf(g_err, sizeof g_err, "bad shape: buckets must be a power of two, row_bytes a "
                                  "multiple of 16, n a multiple of 64");
    return 1;
  }
  release();
  g_shape = Shape{buckets, row_bytes, n};
  const uint64_t slots = buckets * 128;
  CK(hipMalloc((void**)&g_buf.digests, slots));
  CK(hipMalloc((void**)&g_buf.keys, slots * 8));
  CK(hipMalloc((void**)&g_buf.scores, slots * 8));
  CK(hipMalloc((void**)&g_buf.rows, slots * row_bytes));
  CK(hipMalloc((void**)&g_buf.in_rows, n * row_bytes));
  CK(hipMalloc((void**)&g_buf.out_rows, n * row_bytes));
  CK(hipMalloc((void**)&g_buf.in_keys, n * 8));
  CK(hipMalloc((void**)&g_buf.flags, n));
  CK(hipMalloc((void**)&g_buf.small, buckets * 4));
  CK(hipMalloc((void**)&g_buf.sink, 4));
  CK(hipMemset(g_buf.digests, 1, slots));
  CK(hipMemset(g_buf.keys, 2, slots * 8));
  CK(hipMemset(g_buf.scores, 3, slots * 8));
  CK(hipMemset(g_buf.rows, 4, slots * row_bytes));
  CK(hipMemset(g_buf.in_rows, 5, n * row_bytes));
  CK(hipMemset(g_buf.in_keys, 6, n * 8));
  CK(hipMemset(g_buf.small, 0, buckets * 4));
  CK(hipDeviceSynchronize());
  g_ready = true;
  return 0;
}

void hkv_ceilings_release(void) { release(); }

/* Runs pattern `name` once untimed and `reps` times timed (HIP events on the null stream; every
 * launch gets its own salt, so no launch finds the lines of the one before in the caches).
 * `ms` receives the average time of a launch, `bytes` the bytes one launch moves by
 * construction (for the small-access patterns: the number of operations). */
int hkv_ceilings_run(const char* name, int reps, double* ms, double* bytes) {
  if (!g_ready) {
    snprintf(g_err, sizeof g_err, "hkv_ceilings_setup has not been called");
    return 1;
  }
  const Shape sh = g_shape;
  const Buffers b = g_buf;
  const uint64_t n = sh.n;
  const uint32_t upr = sh.row_bytes / 16;
  const uint64_t stream_bytes = n * sh.row_bytes; /* in_rows / out_rows */
  /* the streaming patterns run over pieces of the row region (up to 1 GiB each, another piece
   * for every launch): the dense buffers of a batch are small enough to stay in the caches */
  const uint64_t region = sh.buckets * 128 * sh.row_bytes;
  const uint64_t piece = (region / 8 < (UINT64_C(1) << 30) ? region / 8 : (UINT64_C(1) << 30)) & ~UINT64_C(255);
  const uint64_t piece_units = piece / 16;
  const unsigned row_grid = (unsigned)((n * upr + 255) / 256);
  hipEvent_t e0, e1;
  CK(hipEventCreate(&e0));
  CK(hipEventCreate(&e1));
  double moved = 0;
  /* "step_find" / "step_upsert": the two halves of the benchmark's step, launched in turn,
   * one of them timed launch by launch */
  const bool step_find = !strcmp(name, "step_find"), step_upsert = !strcmp(name, "step_upsert");
  if (step_find || step_upsert) {
    /* three events per step and no synchronisation inside the run, as the benchmark times
     * its own steps */
    hipEvent_t* ev = new hipEvent_t[3 * (reps + 1)];
    for (int q = 0; q < 3 * (reps + 1); q++) CK(hipEventCreate(&ev[q]));
    for (int rep = 0; rep <= reps; rep++) {
      const uint64_t salt = (uint64_t)rep * 0x9E3779B97F4A7C15ULL + 12345;
      CK(hipEventRecord(ev[3 * rep], 0));
      hipLaunchKernelGGL(k_find_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 100u);
      CK(hipEventRecord(ev[3 * rep + 1], 0));
      hipLaunchKernelGGL(k_upsert_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, ~salt, 100u, 1);
      CK(hipEventRecord(ev[3 * rep + 2], 0));
      CK(hipGetLastError());
    }
    CK(hipDeviceSynchronize());
    double sum = 0;
    for (int rep = 1; rep <= reps; rep++) {
      float t = 0;
      CK(hipEventElapsedTime(&t, ev[3 * rep + (step_find ? 0 : 1)], ev[3 * rep + (step_find ? 1 : 2)]));
      sum += t;
    }
    for (int q = 0; q < 3 * (reps + 1); q++) CK(hipEventDestroy(ev[q]));
    delete[] ev;
    CK(hipEventDestroy(e0));
    CK(hipEventDestroy(e1));
    *ms = sum / reps;
    *bytes = step_find ? (double)n * (8 + 128 + 8 + 2.0 * sh.row_bytes + 1)
                       : (double)n * (0.5 * (161 + 2.0 * sh.row_bytes) + 0.5 * (1185 + 2.0 * sh.row_bytes));
    return 0;
  }
  for (int rep = 0; rep <= reps; rep++) {
    const uint64_t salt = (uint64_t)rep * 0x9E3779B97F4A7C15ULL + 12345;
    if (rep == 1) CK(hipEventRecord(e0, 0));
    const u32x4* piece_src = (const u32x4*)(b.rows + (uint64_t)(rep & 3) * piece);
    u32x4* piece_dst = (u32x4*)(b.rows + (uint64_t)(4 + (rep & 3)) * piece);
    if (!strcmp(name, "stream_read")) {
      hipLaunchKernelGGL(k_stream_read, dim3(8192), dim3(256), 0, 0, piece_src, piece_units, b.sink);
      moved = (double)piece;
    } else if (!strcmp(name, "stream_write")) {
      hipLaunchKernelGGL(k_stream_write, dim3(8192), dim3(256), 0, 0, piece_dst, piece_units);
      moved = (double)piece;
    } else if (!strcmp(name, "stream_copy")) {
      hipLaunchKernelGGL(k_stream_copy, dim3(8192), dim3(256), 0, 0, piece_src, piece_dst, piece_units);
      moved = 2.0 * piece;
    } else if (!strcmp(name, "row_gather")) {
      hipLaunchKernelGGL(k_row_gather, dim3(row_grid), dim3(256), 0, 0, sh, b, salt);
      moved = 2.0 * stream_bytes;
    } else if (!strcmp(name, "row_scatter")) {
      hipLaunchKernelGGL(k_row_scatter, dim3(row_grid), dim3(256), 0, 0, sh, b, salt);
      moved = 2.0 * stream_bytes;
    } else if (!strcmp(name, "find_pattern") || !strcmp(name, "find_pattern_1line")) {
      /* 0.44 extra key lines per key: 127 other slots / 256 digest values, 7 of 8 of them in
       * another 128-byte key line; "_1line": exactly one key line per key */
      const uint32_t extra = !strcmp(name, "find_pattern") ? 440 : 0;
      hipLaunchKernelGGL(k_find_pattern<false>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, extra);
      moved = (double)n * (8 + 128 + 8 + 2.0 * sh.row_bytes + 1);
    } else if (!strcmp(name, "find_pattern_chained")) {
      /* 1.1 key lines per key, what the two-step verification fetches */
      hipLaunchKernelGGL(k_find_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 100u);
      moved = (double)n * (8 + 128 + 8 + 2.0 * sh.row_bytes + 1);
    } else if (!strcmp(name, "upsert_pattern_chained")) {
      hipLaunchKernelGGL(k_upsert_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 100u, 1);
      moved = (double)n * (0.5 * (161 + 2.0 * sh.row_bytes) + 0.5 * (1185 + 2.0 * sh.row_bytes));
    } else if (!strcmp(name, "upsert_pattern_free")) {
      hipLaunchKernelGGL(k_upsert_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 50u, 3);
      moved = (double)n * (0.5 * (161 + 2.0 * sh.row_bytes) + 0.5 * (169 + 2.0 * sh.row_bytes));
    } else if (!strcmp(name, "findptr_pattern")) {
      hipLaunchKernelGGL(k_norow_pattern, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 100u, 0);
      moved = (double)n * 153;
    } else if (!strcmp(name, "erase_pattern")) {
      hipLaunchKernelGGL(k_norow_pattern, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 100u, 1);
      moved = (double)n * 165;
    } else if (!strcmp(name, "upsert_pattern_bounds")) {
      hipLaunchKernelGGL(k_upsert_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 100u, 2);
      moved = (double)n * (0.5 * (161 + 2.0 * sh.row_bytes) + 0.5 * (1185 + 2.0 * sh.row_bytes));
    } else if (!strcmp(name, "step_pattern")) {
      /* the benchmark's step: a find and an insert_or_assign on other keys, one after the
       * other, so that each finds the caches as the other left them */
      hipLaunchKernelGGL(k_find_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 100u);
      hipLaunchKernelGGL(k_upsert_pattern<true>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, ~salt, 100u, 1);
      moved = (double)n * (8 + 128 + 8 + 2.0 * sh.row_bytes + 1) +
              (double)n * (0.5 * (161 + 2.0 * sh.row_bytes) + 0.5 * (1185 + 2.0 * sh.row_bytes));
    } else if (!strcmp(name, "upsert_pattern") || !strcmp(name, "upsert_pattern_locks")) {
      const int locks = !strcmp(name, "upsert_pattern_locks");
      hipLaunchKernelGGL(k_upsert_pattern<false>, dim3((unsigned)(n / 64)), dim3(64), 0, 0, sh, b, salt, 440u,
                         locks);
      /* half present (161 + 2 row), half absent into a full bucket (1185 + 2 row) */
      moved = (double)n * (0.5 * (161 + 2.0 * sh.row_bytes) + 0.5 * (1185 + 2.0 * sh.row_bytes));
    } else if (!strncmp(name, "small_", 6)) {
      static const char* kinds[] = {"small_store8", "small_store1", "small_load8", "small_cas64",
                                    "small_xchg64", "small_chunk64", "small_store16", "small_xchg32_side"};
      int kind = -1;
      for (int k = 0; k < 8; k++)
        if (!strcmp(name, kinds[k])) kind = k;
      if (kind < 0) {
        snprintf(g_err, sizeof g_err, "unknown pattern %s", name);
        return 1;
      }
      const uint64_t threads = kind == 5 ? n * 4 : n;
      hipLaunchKernelGGL(k_small, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, 0, sh, b, n, salt,
                         kind);
      moved = (double)n;
    } else {
      snprintf(g_err, sizeof g_err, "unknown pattern %s", name);
      return 1;
    }
    CK(hipGetLastError());
    if (rep == 0) CK(hipDeviceSynchronize());
  }
  CK(hipEventRecord(e1, 0));
  CK(hipEventSynchronize(e1));
  float total = 0;
  CK(hipEventElapsedTime(&total, e0, e1));
  CK(hipEventDestroy(e0));
  CK(hipEventDestroy(e1));
  *ms = (double)total / reps;
  *bytes = moved;
  return 0;
}

}  // extern "C"
