// Exercises the C++ drop-in header the way the reference's own gtest files
// use nv::merlin::HashTable (tests/merlin_hashtable_test.cc.cu:178-423,
// 2674-2849; tests/insert_and_evict_test.cc.cu:34-154;
// tests/export_batch_if_test.cc.cu:128-301; tests/save_and_load_test.cc.cu),
// with a small CHECK macro instead of gtest.  Needs a GPU.
#include <algorithm>
#include <cstdio>
#include <map>
#include <numeric>
#include <random>
#include <set>
#include <unordered_set>
#include <thread>
#include <atomic>
#include <vector>

#include "merlin_hashtable.cuh"
#include "merlin_localfile.hpp"

using namespace nv::merlin;
using K = uint64_t;
using V = float;
using S = uint64_t;

static int g_failures = 0;
#define CHECK(cond)                                                             \
  do {                                                                          \
    if (!(cond)) {                                                              \
      std::printf("CHECK failed %s:%d: %s\n", __FILE__, __LINE__, #cond);       \
      g_failures++;                                                             \
    }                                                                           \
  } while (0)
#define HIP(x) HKV_HIP_CHECK(x)

template <class T>
struct DevBuf {
  T* p = nullptr;
  size_t n = 0;
  explicit DevBuf(size_t n_) : n(n_) { HIP(hipMalloc(reinterpret_cast<void**>(&p), std::max<size_t>(n, 1) * sizeof(T))); }
  ~DevBuf() { (void)hipFree(p); }
  void up(const std::vector<T>& h) { HIP(hipMemcpy(p, h.data(), h.size() * sizeof(T), hipMemcpyHostToDevice)); }
  using H = typename std::conditional<std::is_same<T, bool>::value, uint8_t, T>::type;
  std::vector<H> down(size_t c) const {
    std::vector<H> h(c);
    HIP(hipMemcpy(h.data(), p, c * sizeof(T), hipMemcpyDeviceToHost));
    return h;
  }
};

template <class Kt, class St>
struct ExportIfPredFunctor {
  __forceinline__ __device__ bool operator()(const Kt& key, St& score, const Kt& pattern,
                                             const St& threshold) {
    return score > threshold;
  }
};
template <class Kt, class St>
struct EraseIfPredFunctor {
  __forceinline__ __device__ bool operator()(const Kt& key, St& score, const Kt& pattern,
                                             const St& threshold) {
    return ((key & 0x1u) == 0x1u) && (score > threshold);
  }
};


template <class Kt, class St>
struct MatchNothing {
  __forceinline__ __device__ bool operator()(const Kt&, St&, const Kt&, const St&) { return false; }
};
template <class Kt, class St>
struct MatchEverything {
  __forceinline__ __device__ bool operator()(const Kt&, St&, const Kt&, const St&) { return true; }
};

/* Functors of the tile-cooperative forms, shaped like the ones the reference's tests
 * hand to erase_if_v2 / export_batch_if_v2 / for_each
 * (tests/merlin_hashtable_test.cc.cu:49-97, tests/export_batch_if_test.cc.cu:34-124). */
/* the tile-cooperative export and for_each forms see every slot, free ones included
 * (core_kernels.cuh:1043-1112, 1153-1178): the functor tells them apart */
template <class Kt>
__forceinline__ __device__ bool live_key(const Kt& key) {
  return static_cast<uint64_t>(key) < 0xFFFFFFFFFFFFFFFCull;
}
template <class Kt, class Vt, class St>
struct ScoreBelowV2 {
  St threshold;
  template <int GroupSize>
  __forceinline__ __device__ bool operator()(const Kt& key, const Vt* value, const St& score,
                                             cg::thread_block_tile<GroupSize>& g) {
    return live_key(key) && score < threshold;
  }
};
/* also reads the whole value row, one row at a time by the whole tile */
template <class Kt, class Vt, class St>
struct ScoreBelowAndRowIntactV2 {
  St threshold;
  int dim;
  template <int GroupSize>
  __forceinline__ __device__ bool operator()(const Kt& key, const Vt* value, const St& score,
                                             cg::thread_block_tile<GroupSize>& g) {
    bool mine = live_key(key) && score < threshold;
    for (int r = 0; r < static_cast<int>(g.size()); r++) {
      const Vt* row = g.shfl(value, r);
      const Kt k = g.shfl(key, r);
      const bool candidate = g.shfl(mine, r);
      if (!candidate) continue;
      bool bad = false;
      for (int j = g.thread_rank(); j < dim; j += g.size())
        bad |= row[j] != static_cast<Vt>(static_cast<uint64_t>(k) * 0.00001);
      if (g.ballot(bad) != 0 && static_cast<int>(g.thread_rank()) == r) mine = false;
    }
    return mine;
  }
};
/* for_each body: scales every element of rows whose score is below the
 * threshold, bumps their score by one and counts them */
template <class Kt, class Vt, class St>
struct BumpRowsBelow {
  St threshold;
  int dim;
  Vt factor;
  unsigned long long* counter;
  template <int GroupSize>
  __forceinline__ __device__ void operator()(const Kt& key, Vt* value, St* score,
                                             cg::thread_block_tile<GroupSize>& g) {
    const bool match = live_key(key) && *score < threshold;
    const unsigned long long vote = g.ballot(match);
    if (g.thread_rank() == 0 && vote) atomicAdd(counter, (unsigned long long)__popcll(vote));
    if (match) *score += 1;
    for (int r = 0; r < GroupSize; r++) {
      if (!((vote >> r) & 1ull)) continue;
      Vt* row = g.shfl(value, r);
      for (int j = g.thread_rank(); j < dim; j += GroupSize) row[j] *= factor;
    }
  }
};

static std::vector<K> random_keys(size_t n, uint64_t seed) {
  std::mt19937_64 rng(seed);
  std::unordered_set<K> seen;
  std::vector<K> out;
  while (out.size() < n) {
    K k = rng();
    if ((k & ~UINT64_C(3)) == ~UINT64_C(3)) continue;
    if (seen.insert(k).second) out.push_back(k);
  }
  return out;
}
// v[i][j] = float(key * 0.00001), as tests/test_util.cuh:160-163
static std::vector<V> values_of(const std::vector<K>& keys, size_t dim) {
  std::vector<V> v(keys.size() * dim);
  for (size_t i = 0; i < keys.size(); i++)
    for (size_t j = 0; j < dim; j++) v[i * dim + j] = static_cast<float>(keys[i] * 0.00001);
  return v;
}

static void test_basic() {
  constexpr size_t DIM = 16, N = 1 << 16;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = 64 * 1024 * 1024UL - (128 + 1);
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(16);
  o.reserved_key_start_bit = 2;
  o.num_of_buckets_per_alloc = 32;
  using Table = HashTable<K, V, S, EvictStrategy::kCustomized>;
  Table table;
  table.init(o);
  CHECK(table.bucket_count() == 524287);
  hipStream_t stream;
  HIP(hipStreamCreate(&stream));
  CHECK(table.size(stream) == 0);
  CHECK(table.empty(stream));
  auto keys = random_keys(N, 1);
  auto vals = values_of(keys, DIM);
  std::vector<S> scores(N);
  std::iota(scores.begin(), scores.end(), 1);
  DevBuf<K> dk(N);
  DevBuf<V> dv(N * DIM), dout(N * DIM);
  DevBuf<S> ds(N), dso(N);
  DevBuf<bool> df(N);
  dk.up(keys);
  dv.up(vals);
  ds.up(scores);
  table.insert_or_assign(N, dk.p, dv.p, ds.p, stream);
  CHECK(table.size(stream) == N);
  HIP(hipMemsetAsync(dout.p, 0, N * DIM * sizeof(V), stream));
  table.find(N, dk.p, dout.p, df.p, dso.p, stream);
  HIP(hipStreamSynchronize(stream));
  {
    auto f = df.down(N);
    auto out = dout.down(N * DIM);
    auto so = dso.down(N);
    size_t found = 0;
    bool same = true;
    for (size_t i = 0; i < N; i++) {
      found += f[i];
      same &= so[i] == scores[i];
      for (size_t j = 0; j < DIM; j++) same &= out[i * DIM + j] == vals[i * DIM + j];
    }
    CHECK(found == N);
    CHECK(same);
  }
  // accum_or_assign: existing & flagged -> old + delta
  {
    std::vector<V> delta(vals);  // keys are 64-bit wide, so a small constant would vanish in fp32
    std::vector<char> flags(N, 1);
    DevBuf<V> dd(N * DIM);
    dd.up(delta);
    DevBuf<bool> dflag(N);
    HIP(hipMemcpy(dflag.p, flags.data(), N, hipMemcpyHostToDevice));
    table.accum_or_assign(N, dk.p, dd.p, dflag.p, ds.p, stream);
    table.find(N, dk.p, dout.p, df.p, nullptr, stream);
    HIP(hipStreamSynchronize(stream));
    auto out = dout.down(N * DIM);
    bool same = true;
    for (size_t i = 0; i < N * DIM; i++) same &= out[i] == vals[i] * 2.0f;
    CHECK(same);
  }
  // contains, erase half, clear
  table.contains(N, dk.p, df.p, stream);
  HIP(hipStreamSynchronize(stream));
  {
    auto f = df.down(N);
    CHECK(std::all_of(f.begin(), f.end(), [](uint8_t b) { return b != 0; }));
  }
  table.erase(N / 2, dk.p, stream);
  CHECK(table.size(stream) == N / 2);
  // pointer find on what is left
  {
    DevBuf<V*> dp(N);
    table.find(N, dk.p, dp.p, df.p, nullptr, stream);
    HIP(hipStreamSynchronize(stream));
    auto f = df.down(N);
    auto ptrs = dp.down(N);
    size_t found = 0, nulls = 0;
    for (size_t i = 0; i < N; i++) {
      found += f[i];
      nulls += ptrs[i] == nullptr;
      CHECK(f[i] == (i >= N / 2));
    }
    CHECK(found == N / 2 && nulls == N / 2);
    V row[DIM];
    HIP(hipMemcpy(row, ptrs[N - 1], sizeof row, hipMemcpyDeviceToHost));
    CHECK(row[3] == vals[(N - 1) * DIM + 3] * 2.0f);
  }
  // export == what is resident
  {
    DevBuf<K> ek(N);
    DevBuf<V> ev(N * DIM);
    DevBuf<S> es(N);
    size_t total = 0;
    const size_t cap = table.capacity();
    std::set<K> exported;
    for (size_t off = 0; off < cap; off += 8 * 1024 * 1024) {
      size_t c = table.export_batch(8 * 1024 * 1024, off, ek.p + total, ev.p + total * DIM,
                                    es.p + total, stream);
      total += c;
    }
    CHECK(total == N / 2);
    auto hk = ek.down(total);
    exported.insert(hk.begin(), hk.end());
    CHECK(exported.size() == N / 2);
    for (size_t i = N / 2; i < N; i++) CHECK(exported.count(keys[i]) == 1);
  }
  table.clear(stream);
  CHECK(table.size(stream) == 0);
  CHECK(table.load_factor(stream) == 0.0f);
  HIP(hipStreamDestroy(stream));
}

// keys that land in one bucket (test_util.cuh:296-331), host twin of the hash
static uint64_t fmix64(uint64_t k) {
  k ^= k >> 33;
  k *= UINT64_C(0xff51afd7ed558ccd);
  k ^= k >> 33;
  k *= UINT64_C(0xc4ceb9fe1a85ec53);
  k ^= k >> 33;
  return k;
}
static std::vector<K> keys_in_bucket(size_t n, size_t capacity, size_t bucket, K lo, K hi, uint64_t seed) {
  std::mt19937_64 rng(seed);
  std::unordered_set<K> s;
  std::vector<K> out;
  while (out.size() < n) {
    K c = rng() % (hi - lo) + lo;
    if (((fmix64(c) & (capacity - 1)) / 128) == bucket && s.insert(c).second) out.push_back(c);
  }
  return out;
}

static void test_evict_strategy_customized() {
  constexpr size_t DIM = 4, CAP = 1024;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(1);
  o.reserved_key_start_bit = 15;
  o.num_of_buckets_per_alloc = 8;
  using Table = HashTable<K, V, S, EvictStrategy::kCustomized>;
  auto base = keys_in_bucket(128, CAP, 1, 0, 0x3FFFFFFFFFFFFFFF, 3);
  auto test = keys_in_bucket(128, CAP, 1, 0x3FFFFFFFFFFFFFFF, 0xFFFFFFFFFFFFFFFD, 4);
  for (int i = 64; i < 128; i++) test[i] = base[i];
  std::vector<S> bs(128), ts(128);
  std::iota(bs.begin(), bs.end(), 1000);
  std::iota(ts.begin(), ts.end(), 1128);
  DevBuf<K> dk(128), ek(CAP);
  DevBuf<V> dv(128 * DIM), ev(CAP * DIM);
  DevBuf<S> ds(128), es(CAP);
  for (int rep = 0; rep < 16; rep++) {
    Table table;
    table.init(o);
    dk.up(base);
    dv.up(values_of(base, DIM));
    ds.up(bs);
    table.insert_or_assign(128, dk.p, dv.p, ds.p);
    CHECK(table.size() == 128);
    dk.up(test);
    dv.up(values_of(test, DIM));
    ds.up(ts);
    table.insert_or_assign(128, dk.p, dv.p, ds.p);
    CHECK(table.size() == 128);
    size_t c = table.export_batch(table.capacity(), 0, ek.p, ev.p, es.p);
    CHECK(c == 128);
    auto hs = es.down(c);
    auto hk = ek.down(c);
    auto hv = ev.down(c * DIM);
    std::sort(hs.begin(), hs.end());
    bool ok = true;
    for (size_t i = 0; i < c; i++) ok &= hs[i] == 1128 + i;
    CHECK(ok);
    for (size_t i = 0; i < c; i++) CHECK(hv[i * DIM] == static_cast<float>(hk[i] * 0.00001));
    // scores are required in customized mode (merlin_hashtable.cuh:3846-3850)
    bool threw = false;
    try {
      table.insert_or_assign(128, dk.p, dv.p, nullptr);
    } catch (const MerlinException&) {
      threw = true;
    }
    CHECK(threw);
  }
}

static void test_insert_and_evict_and_predicates() {
  constexpr size_t DIM = 8, CAP = 1 << 16, N = 1 << 14;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(1);
  using Table = HashTable<int64_t, V, S, EvictStrategy::kCustomized>;
  Table table;
  table.init(o);
  std::map<K, V> model;  // key -> first value element, whatever is resident or evicted
  DevBuf<int64_t> dk(N), ek(N);
  DevBuf<V> dv(N * DIM), ev(N * DIM);
  DevBuf<S> ds(N), es(N);
  size_t total_evicted = 0;
  std::map<K, V> resident_or_gone;
  for (int b = 0; b < 8; b++) {  // 8 * 16384 = 2 * capacity fresh keys
    auto keys = random_keys(N, 100 + b);
    auto vals = values_of(keys, DIM);
    std::vector<S> scores(N);
    for (size_t i = 0; i < N; i++) scores[i] = (S(b + 1) << 40) | i;
    std::vector<int64_t> sk(keys.begin(), keys.end());
    dk.up(sk);
    dv.up(vals);
    ds.up(scores);
    size_t before = table.size();
    size_t c = table.insert_and_evict(N, dk.p, dv.p, ds.p, ek.p, ev.p, es.p);
    size_t after = table.size();
    CHECK(c + after == before + N);  // insert_and_evict_test.cc.cu:94,115
    total_evicted += c;
    auto hk = ek.down(c);
    auto hv = ev.down(c * DIM);
    for (size_t i = 0; i < c; i++) CHECK(hv[i * DIM] == static_cast<float>(uint64_t(hk[i]) * 0.00001));
  }
  CHECK(total_evicted > 0);
  CHECK(table.size() <= CAP);
  // size_if == export_batch_if count, every exported tuple satisfies the predicate
  const S threshold = (S(5) << 40);
  size_t expect = table.size_if<ExportIfPredFunctor>(0, threshold);
  DevBuf<int64_t> xk(CAP);
  DevBuf<V> xv(CAP * DIM);
  DevBuf<S> xs(CAP);
  DevBuf<size_t> dc(1);
  table.export_batch_if<ExportIfPredFunctor>(0, threshold, table.capacity(), 0, dc.p, xk.p, xv.p, xs.p);
  HIP(hipDeviceSynchronize());
  size_t got = dc.down(1)[0];
  CHECK(got == expect && got > 0);
  auto hs = xs.down(got);
  CHECK(std::all_of(hs.begin(), hs.end(), [&](S s) { return s > threshold; }));
  auto hk = xk.down(got);
  CHECK(std::set<int64_t>(hk.begin(), hk.end()).size() == got);
  // erase_if removes exactly what size_if counts for the same predicate
  size_t odd_high = table.size_if<EraseIfPredFunctor>(0, threshold);
  size_t before = table.size();
  size_t erased = table.erase_if<EraseIfPredFunctor>(0, threshold);
  CHECK(erased == odd_high);
  CHECK(table.size() == before - erased);
  CHECK(table.size_if<EraseIfPredFunctor>(0, threshold) == 0);
  // the reference's form of size_if: device counter, asynchronous (merlin_hashtable.cuh:3460-3476)
  table.size_if<ExportIfPredFunctor>(0, threshold, dc.p);
  HIP(hipDeviceSynchronize());
  CHECK(dc.down(1)[0] == table.size_if<ExportIfPredFunctor>(0, threshold));
}

struct CountingAllocator : public DefaultAllocator {
  int allocs = 0, frees = 0;
  void alloc(const MemoryType type, void** ptr, size_t size, unsigned int flags = hipHostMallocDefault) override {
    allocs++;
    DefaultAllocator::alloc(type, ptr, size, flags);
  }
  void free(const MemoryType type, void* ptr) override {
    frees++;
    DefaultAllocator::free(type, ptr);
  }
};

static void test_allocator_hybrid_and_checkpoint() {
  constexpr size_t DIM = 32, CAP = 1 << 15, N = 1 << 14;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.max_hbm_for_vectors = CAP * DIM * sizeof(V) / 4;  // a quarter of the rows in HBM
  CountingAllocator alloc;
  auto keys = random_keys(N, 7);
  auto vals = values_of(keys, DIM);
  std::vector<S> scores(N);
  std::iota(scores.begin(), scores.end(), 10);
  DevBuf<K> dk(N);
  DevBuf<V> dv(N * DIM), dout(N * DIM);
  DevBuf<S> ds(N);
  DevBuf<bool> df(N);
  dk.up(keys);
  dv.up(vals);
  ds.up(scores);
  {
    using Table = HashTable<K, V, S, EvictStrategy::kLfu>;
    Table table;
    table.init(o, &alloc);
    CHECK(!table.is_pure_hbm());
    CHECK(alloc.allocs >= 3);
    table.insert_or_assign(N, dk.p, dv.p, ds.p);
    CHECK(table.size() == N);
    table.find(N, dk.p, dout.p, df.p);
    HIP(hipDeviceSynchronize());
    auto out = dout.down(N * DIM);
    CHECK(out == vals);
    // insert_and_evict is refused in hybrid mode (merlin_hashtable.cuh:1384-1386)
    bool threw = false;
    try {
      DevBuf<size_t> dc(1);
      table.insert_and_evict(N, dk.p, dv.p, ds.p, dk.p, dout.p, ds.p, dc.p);
    } catch (const std::runtime_error&) {
      threw = true;
    }
    CHECK(threw);
    // save -> load into a second table
    LocalKVFile<K, V, S> file;
    CHECK(file.open("/tmp/hkv_k.bin", "/tmp/hkv_v.bin", "/tmp/hkv_s.bin", "wb"));
    CHECK(table.save(&file) == N);
    file.close();
    HashTableOptions o2 = o;
    o2.max_hbm_for_vectors = GB(1);
    Table t2;
    t2.init(o2);
    CHECK(file.open("/tmp/hkv_k.bin", "/tmp/hkv_v.bin", "/tmp/hkv_s.bin", "rb"));
    CHECK(t2.load(&file) == N);
    file.close();
    CHECK(t2.size() == N);
    DevBuf<S> dso(N);
    t2.find(N, dk.p, dout.p, df.p, dso.p);
    HIP(hipDeviceSynchronize());
    CHECK(dout.down(N * DIM) == vals);
    CHECK(dso.down(N) == scores);
  }
  CHECK(alloc.allocs == alloc.frees);
}

static void test_option_checks() {
  using Table = HashTable<K, V, S, EvictStrategy::kEpochLru>;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = 1024;
  o.max_hbm_for_vectors = GB(1);
  auto expect_merlin = [&](HashTableOptions bad) {
    bool threw = false;
    try {
      Table t;
      t.init(bad);
    } catch (const MerlinException&) {
      threw = true;
    }
    CHECK(threw);
  };
  HashTableOptions b1 = o;
  b1.reserved_key_start_bit = 63;
  expect_merlin(b1);
  HashTableOptions b2 = o;
  b2.max_bucket_size = 100;
  expect_merlin(b2);
  HashTableOptions b3 = o;
  b3.num_of_buckets_per_alloc = 3;
  expect_merlin(b3);
  Table t;
  t.init(o);
  DevBuf<K> dk(8);
  DevBuf<V> dv(8 * 64);
  bool threw = false;
  try {  // epoch not set (merlin_hashtable.cuh:3853-3860)
    t.insert_or_assign(8, dk.p, dv.p);
  } catch (const MerlinException&) {
    threw = true;
  }
  CHECK(threw);
  t.set_global_epoch(1);
  dk.up(random_keys(8, 5));
  t.insert_or_assign(8, dk.p, dv.p);
  CHECK(t.size() == 8);
  threw = false;
  try {
    t.set_max_capacity(1000);
  } catch (const std::invalid_argument&) {
    threw = true;
  }
  CHECK(threw);
  t.insert_or_assign(0, nullptr, nullptr);  // n == 0 is a no-op
}

/* test_rehash, merlin_hashtable_test.cc.cu:1078-1200, and lock_keys / unlock_keys /
 * find_and_update through the header */
static void test_growth_and_key_locks() {
  constexpr size_t DIM = 16, INIT = 128, MAX = 4 * INIT, N = 2 * INIT;
  HashTableOptions o;
  o.init_capacity = INIT;
  o.max_capacity = MAX;
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(1);
  using Table = HashTable<K, V, S, EvictStrategy::kCustomized>;
  Table table;
  table.init(o);
  CHECK(table.capacity() == INIT);
  /* 64 keys per bucket of the final 4-bucket table: nothing can be evicted */
  std::vector<K> keys;
  for (size_t b = 0; b < 4; b++) {
    auto part = keys_in_bucket(N / 4, MAX, b, 0, 0x3FFFFFFFFFFFFFFF, 11 + b);
    keys.insert(keys.end(), part.begin(), part.end());
  }
  auto vals = values_of(keys, DIM);
  std::vector<S> scores(N);
  for (size_t i = 0; i < N; i++) scores[i] = static_cast<S>(keys[i]);
  DevBuf<K> dk(N);
  DevBuf<V> dv(N * DIM), dout(N * DIM);
  DevBuf<S> ds(N), dso(N);
  DevBuf<bool> df(N);
  dk.up(keys);
  dv.up(vals);
  ds.up(scores);
  table.insert_or_assign(N, dk.p, dv.p, ds.p);  // grows to MAX before the first key goes in
  CHECK(table.capacity() == MAX);
  CHECK(table.size() == N);
  table.reserve(MAX);
  CHECK(table.capacity() == MAX && table.size() == N);
  table.find(N, dk.p, dout.p, df.p, dso.p);
  HIP(hipDeviceSynchronize());
  auto f = df.down(N);
  CHECK(std::all_of(f.begin(), f.end(), [](uint8_t b) { return b != 0; }));
  CHECK(dout.down(N * DIM) == vals);
  CHECK(dso.down(N) == scores);
  table.set_max_capacity(2 * MAX);
  table.reserve(2 * MAX);
  CHECK(table.capacity() == 2 * MAX && table.size() == N);
  table.find(N, dk.p, dout.p, df.p, dso.p);
  HIP(hipDeviceSynchronize());
  CHECK(dout.down(N * DIM) == vals);

  /* lock the first half; locked keys are invisible until unlocked */
  K** dptrs = nullptr;
  HIP(hipMalloc(reinterpret_cast<void**>(&dptrs), N * sizeof(K*)));
  table.lock_keys(N / 2, dk.p, dptrs, df.p, 0, ds.p);
  HIP(hipDeviceSynchronize());
  f = df.down(N / 2);
  CHECK(std::all_of(f.begin(), f.end(), [](uint8_t b) { return b != 0; }));
  table.contains(N, dk.p, df.p);
  HIP(hipDeviceSynchronize());
  f = df.down(N);
  for (size_t i = 0; i < N; i++) CHECK((f[i] != 0) == (i >= N / 2));
  table.unlock_keys(N / 2, dptrs, dk.p, df.p);
  table.contains(N, dk.p, df.p);
  HIP(hipDeviceSynchronize());
  f = df.down(N);
  CHECK(std::all_of(f.begin(), f.end(), [](uint8_t b) { return b != 0; }));
  /* find_and_update: customized scores are replaced by the ones handed in */
  std::vector<S> ns(N);
  for (size_t i = 0; i < N; i++) ns[i] = scores[i] + 7;
  ds.up(ns);
  V** vptrs = nullptr;
  HIP(hipMalloc(reinterpret_cast<void**>(&vptrs), N * sizeof(V*)));
  table.find_and_update(N, dk.p, vptrs, df.p, ds.p);
  table.find(N, dk.p, dout.p, df.p, dso.p);
  HIP(hipDeviceSynchronize());
  CHECK(dso.down(N) == ns);
  (void)hipFree(dptrs);
  (void)hipFree(vptrs);
}


/* The calls whose kernels are compiled in the caller's translation unit (size_if, erase_if,
 * export_batch_if) take the table's layout while they hold their role in the group lock: other
 * host threads that make the table grow meanwhile (which frees the old arrays) must not pull
 * the arrays away under a kernel that is about to be launched.  Four threads insert into a
 * table that grows 64-fold, two keep counting and erasing (a predicate that matches nothing)
 * on streams of their own. */
static void test_header_templates_beside_growth() {
  constexpr size_t DIM = 8, INIT = 1 << 12, MAX = 1 << 18, N = 1024, ROUNDS = 40, WRITERS = 4;
  HashTableOptions o;
  o.init_capacity = INIT;
  o.max_capacity = MAX;
  o.dim = DIM;
  o.max_load_factor = 0.5f;
  o.max_hbm_for_vectors = GB(1);
  using Table = HashTable<K, V, S, EvictStrategy::kLru>;
  Table table;
  table.init(o);
  std::atomic<int> writers_left{(int)WRITERS};
  std::atomic<int> failures{0};
  std::atomic<long> counted{0};
  auto writer = [&](int tid) {
    try {
      hipStream_t st;
      HIP(hipStreamCreate(&st));
      DevBuf<K> dk(N);
      DevBuf<V> dv(N * DIM);
      for (size_t r = 0; r < ROUNDS; r++) {
        std::vector<K> keys(N);
        for (size_t i = 0; i < N; i++) keys[i] = (K)((((uint64_t)tid * ROUNDS + r) * N + i) * 2654435761ull + 17);
        dk.up(keys);
        dv.up(values_of(keys, DIM));
        table.insert_or_assign(N, dk.p, dv.p, nullptr, st);
        HIP(hipStreamSynchronize(st));
      }
      HIP(hipStreamDestroy(st));
    } catch (const std::exception& e) {
      std::printf("writer %d: %s\n", tid, e.what());
      failures++;
    }
    writers_left--;
  };
  auto counter = [&](int tid) {
    try {
      hipStream_t st;
      HIP(hipStreamCreate(&st));
      size_t before = 0;
      while (writers_left.load() > 0) {
        const size_t now = table.template size_if<MatchEverything>(0, 0, st);
        if (now < before || now > WRITERS * ROUNDS * N) failures++;  // keys are never lost or invented
        before = now;
        if (table.template erase_if<MatchNothing>(0, 0, st) != 0) failures++;
        counted++;
      }
      HIP(hipStreamDestroy(st));
    } catch (const std::exception& e) {
      std::printf("counter %d: %s\n", tid, e.what());
      failures++;
    }
  };
  std::vector<std::thread> th;
  for (size_t w = 0; w < WRITERS; w++) th.emplace_back(writer, (int)w);
  for (int c = 0; c < 2; c++) th.emplace_back(counter, c);
  for (auto& x : th) x.join();
  CHECK(failures.load() == 0);
  CHECK(counted.load() > 0);
  CHECK(table.capacity() > INIT);
  CHECK(table.size() == WRITERS * ROUNDS * N);
}

template <size_t DIM>
static void run_functor_forms() {
  constexpr size_t CAP = 1 << 14, N = 6000;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(1);
  using Table = HashTable<int64_t, V, S, EvictStrategy::kCustomized>;
  Table table;
  table.init(o);
  auto keys = random_keys(N, 4242 + DIM);
  auto vals = values_of(keys, DIM);
  std::vector<S> scores(N);
  for (size_t i = 0; i < N; i++) scores[i] = 1000 + i;
  std::vector<int64_t> sk(keys.begin(), keys.end());
  DevBuf<int64_t> dk(N);
  DevBuf<V> dv(N * DIM);
  DevBuf<S> ds(N);
  dk.up(sk);
  dv.up(vals);
  ds.up(scores);
  table.insert_or_assign(N, dk.p, dv.p, ds.p);
  CHECK(table.size() == N);
  std::map<int64_t, size_t> at;
  for (size_t i = 0; i < N; i++) at[sk[i]] = i;
  const S threshold = 1000 + N / 3;

  /* export_batch_if_v2: plain and row-reading predicates agree with the host's count,
   * over the whole table and over two halves */
  DevBuf<int64_t> xk(CAP);
  DevBuf<V> xv(CAP * DIM);
  DevBuf<S> xs(CAP);
  DevBuf<size_t> dc(1);
  auto check_export = [&](size_t got, size_t want) {
    CHECK(got == want);
    auto hk = xk.down(got);
    auto hs = xs.down(got);
    auto hv = xv.down(got * DIM);
    std::set<int64_t> seen;
    bool ok = true;
    for (size_t i = 0; i < got; i++) {
      auto it = at.find(hk[i]);
      if (it == at.end() || hs[i] != scores[it->second] || hs[i] >= threshold) { ok = false; break; }
      for (size_t d = 0; d < DIM; d++) ok &= hv[i * DIM + d] == vals[it->second * DIM + d];
      seen.insert(hk[i]);
    }
    CHECK(ok);
    CHECK(seen.size() == got);
  };
  ScoreBelowV2<int64_t, V, S> below{threshold};
  table.template export_batch_if_v2<ScoreBelowV2<int64_t, V, S>>(below, CAP, 0, dc.p, xk.p, xv.p, xs.p);
  HIP(hipDeviceSynchronize());
  check_export(dc.down(1)[0], N / 3);
  ScoreBelowAndRowIntactV2<int64_t, V, S> intact{threshold, static_cast<int>(DIM)};
  table.template export_batch_if_v2<ScoreBelowAndRowIntactV2<int64_t, V, S>>(intact, CAP, 0, dc.p, xk.p, xv.p, xs.p);
  HIP(hipDeviceSynchronize());
  check_export(dc.down(1)[0], N / 3);
  size_t halves = 0;
  for (size_t off : {size_t(0), CAP / 2}) {
    table.template export_batch_if_v2<ScoreBelowV2<int64_t, V, S>>(below, CAP / 2, off, dc.p, xk.p, xv.p, xs.p);
    HIP(hipDeviceSynchronize());
    halves += dc.down(1)[0];
  }
  CHECK(halves == N / 3);
  table.template export_batch_if_v2<ScoreBelowV2<int64_t, V, S>>(below, CAP, CAP, dc.p, xk.p, xv.p, xs.p);
  HIP(hipDeviceSynchronize());
  CHECK(dc.down(1)[0] == 0);

  /* for_each: rows below the threshold are doubled and get score +1, the others are untouched */
  DevBuf<unsigned long long> cnt(1);
  cnt.up({0ull});
  BumpRowsBelow<int64_t, V, S> bump{threshold, static_cast<int>(DIM), 2.0f, cnt.p};
  table.template for_each<BumpRowsBelow<int64_t, V, S>>(0, table.capacity(), bump);
  HIP(hipDeviceSynchronize());
  CHECK(cnt.down(1)[0] == N / 3);
  DevBuf<V> dout(N * DIM);
  DevBuf<bool> df(N);
  DevBuf<S> dso(N);
  table.find(N, dk.p, dout.p, df.p, dso.p);
  HIP(hipDeviceSynchronize());
  {
    auto out = dout.down(N * DIM);
    auto so = dso.down(N);
    bool ok = true;
    for (size_t i = 0; i < N; i++) {
      const bool hit = scores[i] < threshold;
      ok &= so[i] == scores[i] + (hit ? 1 : 0);
      for (size_t d = 0; d < DIM; d++) ok &= out[i * DIM + d] == vals[i * DIM + d] * (hit ? 2.0f : 1.0f);
    }
    CHECK(ok);
  }
  /* the bumped rows no longer pass the row-reading predicate; the plain one sees the
   * new scores (one key moved across the threshold) */
  size_t erased = table.template erase_if_v2<ScoreBelowAndRowIntactV2<int64_t, V, S>>(intact);
  CHECK(erased == 0);
  CHECK(table.size() == N);
  erased = table.template erase_if_v2<ScoreBelowV2<int64_t, V, S>>(below);
  CHECK(erased == N / 3 - 1);
  CHECK(table.size() == N - erased);
  table.contains(N, dk.p, df.p);
  HIP(hipDeviceSynchronize());
  {
    auto f = df.down(N);
    bool ok = true;
    for (size_t i = 0; i < N; i++) ok &= (f[i] != 0) == !(scores[i] + 1 < threshold);
    CHECK(ok);
  }
  /* erased slots are reusable */
  table.insert_or_assign(N, dk.p, dv.p, ds.p);
  CHECK(table.size() == N);
}

static void test_functor_forms() {
  run_functor_forms<64>();  // tiles of 32
  run_functor_forms<16>();  // tiles of 16
  run_functor_forms<8>();   // tiles of 8
  run_functor_forms<3>();   // one thread per slot
}


/* for_each body that pushes the scores of odd keys down to 1..N: what a caller may do with the
 * writable score it is handed */
template <class Kt, class Vt, class St>
struct SinkOddKeys {
  template <int GroupSize>
  __forceinline__ __device__ void operator()(const Kt& key, Vt* value, St* score,
                                             cg::thread_block_tile<GroupSize>& g) {
    if (live_key(key) && (key & 1u)) *score = 1 + (static_cast<uint64_t>(key) >> 40);
  }
};

/* An LRU table finds eviction victims through per-line lower bounds of the scores
 * (hkv_table_view::bounds).  The calls of the header that change slots or scores behind the
 * library's back - erase_if, erase_if_v2 and for_each with a functor that writes scores - must
 * leave them right: after each, and after upserts that evict, no bound is above a
 * score of its line, and the keys whose scores were pushed down are the ones that go. */
static void test_score_bounds_after_header_calls() {
  constexpr size_t DIM = 8, CAP = 1 << 14, N = 1 << 13;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(1);
  using Table = HashTable<K, V, S, EvictStrategy::kLru>;
  Table table;
  table.init(o);
  auto bounds_hold = [&]() {
    HIP(hipDeviceSynchronize());
    hkv_table_view v;
    if (hkv_table_get_view(table.native_handle(), &v)) return false;
    if (!v.bounds) return true;  // HKV_SCORE_BOUNDS=0: nothing to hold
    std::vector<uint64_t> sc(v.capacity), ks(v.capacity), bd(v.capacity / 16);
    HIP(hipMemcpy(sc.data(), v.scores, sc.size() * 8, hipMemcpyDeviceToHost));
    HIP(hipMemcpy(ks.data(), v.keys, ks.size() * 8, hipMemcpyDeviceToHost));
    HIP(hipMemcpy(bd.data(), v.bounds, bd.size() * 8, hipMemcpyDeviceToHost));
    for (size_t l = 0; l < bd.size(); l++)
      for (size_t q = 0; q < 16; q++)  // a free slot gets its score when it is taken
        if (ks[l * 16 + q] != v.empty_key && bd[l] > sc[l * 16 + q]) return false;
    return true;
  };
  DevBuf<K> dk(N);
  DevBuf<V> dv(N * DIM);
  auto put = [&](uint64_t seed) {
    auto keys = random_keys(N, seed);
    dk.up(keys);
    dv.up(values_of(keys, DIM));
    table.insert_or_assign(N, dk.p, dv.p);
    return keys;
  };
  for (uint64_t b = 0; b < 5; b++) put(4000 + b);  // 2.5 x capacity: every bucket has evicted
  CHECK(table.size() > CAP * 95 / 100);
  CHECK(bounds_hold());
  // slots freed by both erase_if forms, in lines whose bounds are tight
  const size_t before = table.size();
  const size_t odd = table.template erase_if<EraseIfPredFunctor>(0, S(0));  // odd keys, any score
  CHECK(odd > before / 3 && table.size() == before - odd);
  CHECK(bounds_hold());
  put(4010);
  CHECK(bounds_hold());
  ScoreBelowV2<K, V, S> all{~S(0)};
  const size_t rest = table.template erase_if_v2<ScoreBelowV2<K, V, S>>(all);
  CHECK(rest > 0 && table.size() == 0);
  CHECK(bounds_hold());
  // refill, then push the scores of the odd keys far down through for_each: they go first
  std::vector<K> resident;
  for (uint64_t b = 0; b < 4; b++) {
    auto k = put(4020 + b);
    resident.insert(resident.end(), k.begin(), k.end());
  }
  SinkOddKeys<K, V, S> sink;
  table.template for_each<SinkOddKeys<K, V, S>>(0, table.capacity(), sink);
  HIP(hipDeviceSynchronize());
  CHECK(table.template size_if<EraseIfPredFunctor>(0, S(0)) > CAP / 3);
  hkv_table_view v;
  CHECK(hkv_table_get_view(table.native_handle(), &v) == 0);
  std::vector<uint64_t> keys0(v.capacity), keys1(v.capacity), sc1(v.capacity);
  HIP(hipMemcpy(keys0.data(), v.keys, keys0.size() * 8, hipMemcpyDeviceToHost));
  put(4030);  // a table's worth of new keys: every eviction takes its bucket's lowest score
  put(4031);
  CHECK(bounds_hold());
  HIP(hipMemcpy(keys1.data(), v.keys, keys1.size() * 8, hipMemcpyDeviceToHost));
  HIP(hipMemcpy(sc1.data(), v.scores, sc1.size() * 8, hipMemcpyDeviceToHost));
  /* bucket by bucket: while a sunk score is left in a bucket, no key that was not sunk can have
   * been evicted from it */
  size_t wrong = 0, sunk_gone = 0;
  for (size_t b = 0; b < v.buckets_num; b++) {
    std::unordered_set<uint64_t> after(keys1.begin() + b * 128, keys1.begin() + (b + 1) * 128);
    bool sunk_left = false, even_lost = false;
    for (size_t q = 0; q < 128; q++) {
      const uint64_t k1 = keys1[b * 128 + q], k0 = keys0[b * 128 + q];
      if (k1 < 0xFFFFFFFFFFFFFFFCull && (k1 & 1u) && sc1[b * 128 + q] < (1ull << 30)) sunk_left = true;
      if (k0 < 0xFFFFFFFFFFFFFFFCull && !after.count(k0)) {
        if (k0 & 1u)
          sunk_gone++;
        else
          even_lost = true;
      }
    }
    if (sunk_left && even_lost) wrong++;
  }
  CHECK(wrong == 0);
  CHECK(sunk_gone > CAP / 4);
}

// TableMode::kMemory through the header: init checks, insert_or_assign + find, guards
// (tests/dual_bucket_test.cc.cu:74-158, 471-515, 641-661, 1051-1107)
static void test_dual_bucket_mode() {
  constexpr size_t DIM = 16, CAP = 128 * 128, N = 8000;
  using Table = HashTable<K, V, S, EvictStrategy::kCustomized>;
  auto make = [&](size_t init, size_t max, size_t hbm, size_t dim) {
    HashTableOptions o;
    o.init_capacity = init;
    o.max_capacity = max;
    o.max_hbm_for_vectors = hbm;
    o.dim = dim;
    o.table_mode = TableMode::kMemory;
    return o;
  };
  auto rejects = [&](const HashTableOptions& o) {
    Table t;
    try {
      t.init(o);
    } catch (const std::exception&) {
      return true;
    }
    return false;
  };
  CHECK(rejects(make(CAP, 2 * CAP, 0, DIM)));
  CHECK(rejects(make(CAP, CAP, GB(1), DIM)));
  CHECK(rejects(make(CAP, CAP, 0, 225)));
  CHECK(rejects(make(128, 128, 0, DIM)));
  Table table;
  table.init(make(CAP, CAP, 0, DIM));
  auto keys = random_keys(N, 99);
  auto vals = values_of(keys, DIM);
  std::vector<S> scores(N);
  for (size_t i = 0; i < N; i++) scores[i] = 10 + i;
  DevBuf<K> dk(N);
  DevBuf<V> dv(N * DIM), dout(N * DIM);
  DevBuf<S> ds(N), dso(N);
  DevBuf<bool> df(N);
  dk.up(keys);
  dv.up(vals);
  ds.up(scores);
  table.insert_or_assign(N, dk.p, dv.p, ds.p);
  CHECK(table.size() == N);
  table.find(N, dk.p, dout.p, df.p, dso.p);
  HIP(hipDeviceSynchronize());
  auto f = df.down(N);
  CHECK(std::all_of(f.begin(), f.end(), [](uint8_t b) { return b != 0; }));
  CHECK(dout.down(N * DIM) == vals);
  CHECK(dso.down(N) == scores);
  int threw = 0;
  auto expect_throw = [&](auto&& call) {
    try {
      call();
    } catch (const std::exception&) {
      threw++;
    }
  };
  expect_throw([&] { table.erase(N, dk.p); });
  expect_throw([&] { table.contains(N, dk.p, df.p); });
  expect_throw([&] { table.reserve(2 * CAP); });
  expect_throw([&] { table.find_or_insert(N, dk.p, dout.p, ds.p); });
  expect_throw([&] { table.assign_scores(N, dk.p, ds.p); });
  expect_throw([&] { table.assign_values(N, dk.p, dv.p); });
  expect_throw([&] { table.insert_or_assign(N, dk.p, dv.p, ds.p, 0, false); });
  CHECK(threw == 7);
  CHECK(table.size() == N);
  table.clear();
  CHECK(table.size() == 0);
}


// io_by_cpu (tests/merlin_hashtable_test.cc.cu:1760-1905, test_basic_for_cpu_io): every row in
// pinned host memory, the rows of the writers moved by host threads; the same sequence of calls
// and counts, plus a check of the rows the reference's test leaves out.
static void test_basic_for_cpu_io() {
  constexpr size_t DIM = 16, CAP = 1 << 20, N = 1 << 16;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.reserved_key_start_bit = 10;
  o.max_hbm_for_vectors = GB(0);
  o.io_by_cpu = true;
  using Table = HashTable<K, V, S, EvictStrategy::kCustomized>;
  {
    HashTableOptions bad = o;
    bad.max_hbm_for_vectors = GB(1);  // merlin_hashtable.cuh:1071-1073
    Table t;
    bool threw = false;
    try {
      t.init(bad);
    } catch (const MerlinException&) {
      threw = true;
    }
    CHECK(threw);
  }
  Table table;
  table.init(o);
  hipStream_t stream;
  HIP(hipStreamCreate(&stream));
  CHECK(table.size(stream) == 0);
  std::vector<K> keys;
  {
    // the reserved keys sit at bit 10 on this table (types.cuh:80-109)
    std::mt19937_64 rng(77);
    std::unordered_set<K> seen;
    const K mask = ~(UINT64_C(3) << 10) & ~UINT64_C(1);
    while (keys.size() < N) {
      K k = rng();
      if ((k & mask) == mask) continue;
      if (seen.insert(k).second) keys.push_back(k);
    }
  }
  std::vector<S> scores(N);
  std::iota(scores.begin(), scores.end(), 1);
  std::vector<V> ones(N * DIM, 1.0f), twos(N * DIM, 2.0f);
  DevBuf<K> dk(N), dko(CAP);
  DevBuf<V> dv(N * DIM), dout(N * DIM), dvo(CAP * DIM);
  DevBuf<S> ds(N), dso(CAP);
  DevBuf<bool> df(N);
  dk.up(keys);
  ds.up(scores);
  dv.up(ones);
  table.insert_or_assign(N, dk.p, dv.p, ds.p, stream);
  CHECK(table.size(stream) == N);
  dv.up(twos);
  table.insert_or_assign(N, dk.p, dv.p, ds.p, stream);
  CHECK(table.size(stream) == N);
  table.find(N, dk.p, dout.p, df.p, nullptr, stream);
  HIP(hipStreamSynchronize(stream));
  {
    auto f = df.down(N);
    auto out = dout.down(N * DIM);
    size_t found = 0;
    bool same = true;
    for (size_t i = 0; i < N; i++) found += f[i];
    for (size_t i = 0; i < N * DIM; i++) same &= out[i] == 2.0f;
    CHECK(found == N);
    CHECK(same);
  }
  HIP(hipMemsetAsync(df.p, 0, N, stream));
  table.contains(N, dk.p, df.p, stream);
  HIP(hipStreamSynchronize(stream));
  {
    auto f = df.down(N);
    size_t n = 0;
    for (size_t i = 0; i < N; i++) n += f[i];
    CHECK(n == N);
  }
  table.accum_or_assign(N, dk.p, dv.p, df.p, ds.p, stream);  // every flag says accumulate: 2 + 2
  CHECK(table.size(stream) == N);
  // find_or_insert: the first half is there (rows come back), the second half is new
  {
    auto more = random_keys(N / 2, 78);
    std::vector<K> mixed(keys.begin(), keys.begin() + N / 2);
    mixed.insert(mixed.end(), more.begin(), more.end());
    DevBuf<K> dm(N);
    dm.up(mixed);
    std::vector<V> io(N * DIM, 7.0f);
    DevBuf<V> dio(N * DIM);
    dio.up(io);
    table.find_or_insert(N, dm.p, dio.p, ds.p, stream);
    HIP(hipStreamSynchronize(stream));
    auto back = dio.down(N * DIM);
    bool same = true;
    for (size_t i = 0; i < N / 2 * DIM; i++) same &= back[i] == 4.0f;
    for (size_t i = N / 2 * DIM; i < N * DIM; i++) same &= back[i] == 7.0f;
    CHECK(same);
    CHECK(table.size(stream) == N + N / 2);
    table.assign_values(N / 2, dm.p + N / 2, dv.p, stream);  // the new keys get rows of 2.0
    table.find(N, dm.p, dout.p, df.p, nullptr, stream);
    HIP(hipStreamSynchronize(stream));
    auto out = dout.down(N * DIM);
    same = true;
    for (size_t i = 0; i < N / 2 * DIM; i++) same &= out[i] == 4.0f;
    for (size_t i = N / 2 * DIM; i < N * DIM; i++) same &= out[i] == 2.0f;
    CHECK(same);
    table.erase(N / 2, dm.p + N / 2, stream);
  }
  table.erase(N >> 1, dk.p, stream);
  CHECK(table.size(stream) == N >> 1);
  table.clear(stream);
  CHECK(table.size(stream) == 0);
  table.insert_or_assign(N, dk.p, dv.p, ds.p, stream);
  size_t dumped = table.export_batch(table.capacity(), 0, dko.p, dvo.p, dso.p, stream);
  HIP(hipStreamSynchronize(stream));
  CHECK(dumped == N);
  HIP(hipStreamDestroy(stream));
}

// save -> load into a second table, for every strategy (tests/save_and_load_test.cc.cu:30-120):
// the tables hold the same keys and rows afterwards, and the same scores where the caller
// supplies them (LRU and EpochLRU scores are clock readings of the loading call).
template <class Table>
static std::map<K, std::pair<std::vector<V>, S>> table_contents(Table& t, size_t dim) {
  const size_t cap = t.capacity();
  DevBuf<K> dk(cap);
  DevBuf<V> dv(cap * dim);
  DevBuf<S> ds(cap);
  const size_t n = t.export_batch(cap, 0, dk.p, dv.p, ds.p);
  auto k = dk.down(n);
  auto v = dv.down(n * dim);
  auto sc = ds.down(n);
  std::map<K, std::pair<std::vector<V>, S>> m;
  for (size_t i = 0; i < n; i++)
    m[k[i]] = {std::vector<V>(v.begin() + i * dim, v.begin() + (i + 1) * dim), sc[i]};
  return m;
}
template <int Strategy>
static void run_save_and_load() {
  constexpr size_t DIM = 8, CAP = 1 << 17, N = 1 << 16;
  using Table = HashTable<K, V, S, Strategy>;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(1);
  auto keys = random_keys(N, 500 + Strategy);
  auto vals = values_of(keys, DIM);
  std::vector<S> scores(N);
  std::iota(scores.begin(), scores.end(), 1000);
  DevBuf<K> dk(N);
  DevBuf<V> dv(N * DIM);
  DevBuf<S> ds(N);
  dk.up(keys);
  dv.up(vals);
  ds.up(scores);
  Table t0, t1;
  t0.init(o);
  t1.init(o);
  constexpr bool clocked = Strategy == EvictStrategy::kLru || Strategy == EvictStrategy::kEpochLru;
  t0.set_global_epoch(101);
  t0.insert_or_assign(N, dk.p, dv.p, clocked ? nullptr : ds.p);
  CHECK(t0.size() == N);
  LocalKVFile<K, V, S> file;
  CHECK(file.open("/tmp/hkv_sl_k.bin", "/tmp/hkv_sl_v.bin", "/tmp/hkv_sl_s.bin", "wb"));
  CHECK(t0.save(&file, 64 * 1024) == N);  // a small work space: many windows
  file.close();
  CHECK(file.open("/tmp/hkv_sl_k.bin", "/tmp/hkv_sl_v.bin", "/tmp/hkv_sl_s.bin", "rb"));
  CHECK(t1.load(&file, 48 * 1024) == N);
  file.close();
  auto a = table_contents(t0, DIM), b = table_contents(t1, DIM);
  CHECK(a.size() == N && b.size() == N);
  bool same = a.size() == b.size();
  for (auto& kv : a) {
    auto it = b.find(kv.first);
    if (it == b.end() || it->second.first != kv.second.first) {
      same = false;
      break;
    }
    if (it->second.second != kv.second.second) same = false;  // load keeps the saved scores
  }
  CHECK(same);
}
static void test_save_and_load_all_strategies() {
  run_save_and_load<EvictStrategy::kLru>();
  run_save_and_load<EvictStrategy::kLfu>();
  run_save_and_load<EvictStrategy::kEpochLru>();
  run_save_and_load<EvictStrategy::kEpochLfu>();
  run_save_and_load<EvictStrategy::kCustomized>();
}

// S = uint32_t (tests/uint32_score_test.cc.cu:48-186): find_or_insert + find return the
// 32-bit scores handed in, missing keys leave the caller's score entries alone,
// assign_scores + export_batch round-trip, insert_and_evict hands back 32-bit scores.
static void test_uint32_scores() {
  using S32 = uint32_t;
  using Table = HashTable<K, V, S32, EvictStrategy::kCustomized>;
  constexpr size_t DIM = 16, CAP = 1 << 15, N = 4096;
  HashTableOptions o;
  o.init_capacity = o.max_capacity = CAP;
  o.dim = DIM;
  o.max_hbm_for_vectors = GB(1);
  Table table;
  table.init(o);
  auto keys = random_keys(N, 321);
  auto vals = values_of(keys, DIM);
  std::vector<S32> scores(N);
  for (size_t i = 0; i < N; i++) scores[i] = 1000u + static_cast<S32>(i) * 3u;
  DevBuf<K> dk(N);
  DevBuf<V> dv(N * DIM), dout(N * DIM);
  DevBuf<S32> ds(N), dso(N);
  DevBuf<bool> df(N);
  dk.up(keys);
  dv.up(vals);
  ds.up(scores);
  table.find_or_insert(N, dk.p, dv.p, ds.p);
  CHECK(table.size() == N);
  table.find(N, dk.p, dout.p, df.p, dso.p);
  HIP(hipDeviceSynchronize());
  auto f = df.down(N);
  CHECK(std::all_of(f.begin(), f.end(), [](uint8_t b) { return b != 0; }));
  CHECK(dso.down(N) == scores);
  CHECK(dout.down(N * DIM) == vals);
  // missing keys: founds false, the score entries keep the caller's sentinel
  auto missing = random_keys(N, 654);
  DevBuf<K> dm(N);
  dm.up(missing);
  std::vector<S32> sentinel(N, 0xDEADBEEFu);
  dso.up(sentinel);
  table.find(N, dm.p, dout.p, df.p, dso.p);
  HIP(hipDeviceSynchronize());
  f = df.down(N);
  CHECK(std::none_of(f.begin(), f.end(), [](uint8_t b) { return b != 0; }));
  CHECK(dso.down(N) == sentinel);
  // assign_scores, then export everything
  for (size_t i = 0; i < N; i++) scores[i] = 500000u + static_cast<S32>(N - i);
  ds.up(scores);
  table.assign_scores(N, dk.p, ds.p);
  DevBuf<K> xk(CAP);
  DevBuf<V> xv(CAP * DIM);
  DevBuf<S32> xs(CAP);
  const size_t dumped = table.export_batch(table.capacity(), 0, xk.p, xv.p, xs.p);
  CHECK(dumped == N);
  {
    std::map<K, S32> want;
    for (size_t i = 0; i < N; i++) want[keys[i]] = scores[i];
    auto hk = xk.down(dumped);
    auto hs = xs.down(dumped);
    bool ok = true;
    for (size_t i = 0; i < dumped; i++) {
      auto it = want.find(hk[i]);
      ok &= it != want.end() && it->second == hs[i];
      if (it != want.end()) want.erase(it);
    }
    CHECK(ok && want.empty());
  }
  // fill one bucket's worth of pressure: insert_and_evict returns 32-bit scores of what left
  constexpr size_t M = 1 << 15;
  auto more = random_keys(M, 987);
  auto mvals = values_of(more, DIM);
  std::vector<S32> mscores(M);
  for (size_t i = 0; i < M; i++) mscores[i] = 2000000u + static_cast<S32>(i);
  DevBuf<K> mk(M), ek(M);
  DevBuf<V> mv(M * DIM), ev(M * DIM);
  DevBuf<S32> ms(M), es(M);
  mk.up(more);
  mv.up(mvals);
  ms.up(mscores);
  const size_t before = table.size();
  const size_t c = table.insert_and_evict(M, mk.p, mv.p, ms.p, ek.p, ev.p, es.p);
  CHECK(c + table.size() == before + M);
  CHECK(c > 0);
  {
    std::map<K, S32> old;
    for (size_t i = 0; i < N; i++) old[keys[i]] = scores[i];
    for (size_t i = 0; i < M; i++) old[more[i]] = mscores[i];
    auto hk = ek.down(c);
    auto hs = es.down(c);
    bool ok = true;
    for (size_t i = 0; i < c; i++) ok &= old.count(hk[i]) == 1 && old[hk[i]] == hs[i];
    CHECK(ok);
  }
  // a predicate over 32-bit scores
  const size_t high = table.size_if<ExportIfPredFunctor>(0, static_cast<S32>(2000000u - 1));
  CHECK(high > 0 && high <= M);
}

int main() {
  try {
    test_basic();
    test_evict_strategy_customized();
    test_insert_and_evict_and_predicates();
    test_allocator_hybrid_and_checkpoint();
    test_option_checks();
    test_growth_and_key_locks();
    test_header_templates_beside_growth();
    test_functor_forms();
    test_score_bounds_after_header_calls();
    test_dual_bucket_mode();
    test_uint32_scores();
    test_basic_for_cpu_io();
    test_save_and_load_all_strategies();
  } catch (const std::exception& e) {
    std::printf("unexpected exception: %s\n", e.what());
    return 2;
  }
  if (g_failures) {
    std::printf("%d checks failed\n", g_failures);
    return 1;
  }
  std::printf("api_test: all checks passed\n");
  return 0;
}
