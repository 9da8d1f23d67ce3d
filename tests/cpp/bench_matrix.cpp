// The reference's benchmark table through the drop-in C++ header: one timed call of 2^20 keys per
// API at load factors 0.50 / 0.75 / 1.00 and dim 8 / 32 / 64, LRU, in units of 2^30 KV/s.
// Protocol after benchmark/merlin_hashtable_benchmark.cc.cu:75-420 and benchmark_util.cuh:135-177:
// consecutive integer keys up to the load factor, 60 % of a call's keys from the last inserted
// batch and 40 % never seen, host clock from the call to the end of the stream, best of two.
// One table per (dim, load factor) serves all APIs, the read-only ones first.
//
//   tests/cpp/bench_matrix            pure HBM rows of the table
//   tests/cpp/bench_matrix --hybrid   dim 64, capacity 128M, 16 GB of the rows in HBM
#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <numeric>
#include <string>
#include <vector>

#include "merlin_hashtable.cuh"

using namespace nv::merlin;
using K = uint64_t;
using V = float;
using S = uint64_t;
using Table = HashTable<K, V, S, EvictStrategy::kLru>;

#define HIP(x) HKV_HIP_CHECK(x)

template <class Kt, class St>
struct ScoreAbove {
  __forceinline__ __device__ bool operator()(const Kt& key, St& score, const Kt& pattern,
                                             const St& threshold) {
    return score > threshold;
  }
};

template <class T>
static T* dev_alloc(size_t n) {
  T* p = nullptr;
  HIP(hipMalloc(reinterpret_cast<void**>(&p), std::max<size_t>(n, 1) * sizeof(T)));
  return p;
}

__global__ void iota_kernel(K* keys, size_t n, K first, long long step) {
  const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  if (i < n) keys[i] = first + (K)((long long)i * step);
}
static void fill_keys(K* d, size_t n, K first, long long step, hipStream_t s) {
  if (n) hipLaunchKernelGGL(iota_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, d, n, first, step);
}
__global__ void fill_rows_kernel(V* rows, size_t n, V x) {
  const size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x;
  if (i < n) rows[i] = x;
}

int main(int argc, char** argv) {
  const bool hybrid = argc > 1 && !strcmp(argv[1], "--hybrid");
  const size_t n = 1 << 20, M = 1 << 20;
  struct Config {
    size_t dim, cap, hbm;
  };
  std::vector<Config> configs;
  if (hybrid)
    configs = {{64, 128 * M, GB(16)}};
  else
    configs = {{8, 128 * M, GB(4)}, {32, 128 * M, GB(16)}, {64, 64 * M, GB(16)}};
  std::vector<std::string> apis = {"insert_or_assign", "find",   "find_or_insert",  "assign",
                                   "find*",            "find_or_insert*", "insert_and_evict",
                                   "export_batch",     "export_batch_if", "contains"};
  std::vector<std::string> order = {"find",   "find*",          "contains",        "export_batch",
                                    "export_batch_if", "assign", "find_or_insert",  "find_or_insert*",
                                    "insert_or_assign", "insert_and_evict"};
  if (hybrid) {  // insert_and_evict needs a pure-HBM table (merlin_hashtable.cuh:1373-1375)
    apis.erase(std::find(apis.begin(), apis.end(), "insert_and_evict"));
    order.erase(std::find(order.begin(), order.end(), "insert_and_evict"));
  }
  std::printf("| dim | capacity | HBM for rows | load factor |");
  for (auto& a : apis) std::printf(" %s |", a.c_str());
  std::printf("\n|---|---|---|---|");
  for (size_t i = 0; i < apis.size(); i++) std::printf("---|");
  std::printf("\n");
  hipStream_t stream;
  HIP(hipStreamCreate(&stream));
  try {
    for (const Config& c : configs) {
      const size_t max_out = (size_t)(n / 0.5) + 16;
      K* d_keys = dev_alloc<K>(max_out);
      V* d_vals = dev_alloc<V>(max_out * c.dim);
      V* d_def = dev_alloc<V>(n * c.dim);
      V** d_ptrs = dev_alloc<V*>(n);
      bool* d_found = dev_alloc<bool>(n);
      K* d_ek = dev_alloc<K>(n);
      S* d_es = dev_alloc<S>(n);
      size_t* d_cnt = dev_alloc<size_t>(1);
      hipLaunchKernelGGL(fill_rows_kernel, dim3((unsigned)((max_out * c.dim + 255) / 256)), dim3(256), 0, stream,
                         d_vals, max_out * c.dim, 1.0f);
      hipLaunchKernelGGL(fill_rows_kernel, dim3((unsigned)((n * c.dim + 255) / 256)), dim3(256), 0, stream, d_def,
                         n * c.dim, 2.0f);
      for (double lf : {0.50, 0.75, 1.00}) {
        HashTableOptions o;
        o.init_capacity = o.max_capacity = c.cap;
        o.max_hbm_for_vectors = c.hbm;
        o.dim = c.dim;
        Table table;
        table.init(o);
        size_t start = 0;
        const size_t target = (size_t)(c.cap * lf);
        while (start < target) {
          const size_t m = std::min(n, target - start);
          fill_keys(d_keys, m, start, 1, stream);
          table.insert_or_assign(m, d_keys, d_vals, nullptr, stream);
          start += m;
        }
        while (true) {  // top up: buckets that overflowed have evicted
          const size_t size = table.size(stream);
          if (size + c.cap / 1000 >= target || start > 3 * c.cap) break;
          const size_t m = std::min(n, target - size);
          fill_keys(d_keys, m, start, 1, stream);
          table.insert_or_assign(m, d_keys, d_vals, nullptr, stream);
          start += m;
        }
        std::vector<double> res(apis.size(), 0.0);
        K fresh = ~K(0) - 4;  // never-seen keys count down from the top, below the reserved ones
        const size_t n_hit = (size_t)(n * 0.6), n_new = n - n_hit;
        const size_t n_export = (size_t)(n / lf * 0.995);
        for (auto& api : order) {
          double best = 1e30;
          for (int rep = 0; rep < 2; rep++) {
            fill_keys(d_keys, n_hit, start - n, 1, stream);
            fill_keys(d_keys + n_hit, n_new, fresh, -1, stream);
            fresh -= n_new;
            HIP(hipMemsetAsync(d_cnt, 0, sizeof(size_t), stream));
            HIP(hipStreamSynchronize(stream));
            const auto t0 = std::chrono::steady_clock::now();
            if (api == "find")
              table.find(n, d_keys, d_vals, d_found, nullptr, stream);
            else if (api == "find*")
              table.find(n, d_keys, d_ptrs, d_found, nullptr, stream);
            else if (api == "contains")
              table.contains(n, d_keys, d_found, stream);
            else if (api == "export_batch")
              table.export_batch(n_export, 0, d_cnt, d_keys, d_vals, nullptr, stream);
            else if (api == "export_batch_if")
              table.export_batch_if<ScoreAbove>(0, 0, n_export, 0, d_cnt, d_keys, d_vals, nullptr, stream);
            else if (api == "assign")
              table.assign(n, d_keys, d_def, nullptr, stream);
            else if (api == "find_or_insert")
              table.find_or_insert(n, d_keys, d_vals, nullptr, stream);
            else if (api == "find_or_insert*")
              table.find_or_insert(n, d_keys, d_ptrs, d_found, nullptr, stream);
            else if (api == "insert_or_assign")
              table.insert_or_assign(n, d_keys, d_vals, nullptr, stream);
            else if (api == "insert_and_evict")
              table.insert_and_evict(n, d_keys, d_vals, nullptr, d_ek, d_def, d_es, d_cnt, stream);
            HIP(hipStreamSynchronize(stream));
            const double sec = std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count();
            best = std::min(best, sec);
          }
          res[std::find(apis.begin(), apis.end(), api) - apis.begin()] = n / best / double(1 << 30);
        }
        std::printf("| %zu | %zuM | %zu GB | %.2f |", c.dim, c.cap / M, c.hbm >> 30,
                    (double)table.size(stream) / c.cap);
        for (double r : res) std::printf(" %.3f |", r);
        std::printf("\n");
        std::fflush(stdout);
      }
      for (void* p : {(void*)d_keys, (void*)d_vals, (void*)d_def, (void*)d_ptrs, (void*)d_found, (void*)d_ek,
                      (void*)d_es, (void*)d_cnt})
        (void)hipFree(p);
    }
  } catch (const std::exception& e) {
    std::printf("exception: %s\n", e.what());
    return 2;
  }
  HIP(hipStreamDestroy(stream));
  return 0;
}
