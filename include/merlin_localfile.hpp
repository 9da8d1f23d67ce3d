/*
 * LocalKVFile: BaseKVFile over three flat little-endian files (keys, values,
 * scores), the checkpoint format of the reference (include/merlin_localfile.hpp:
 * 61-151): keys as K[n], values as V[n * dim], scores as S[n].
 */
#ifndef MERLIN_LOCALFILE_HPP_
#define MERLIN_LOCALFILE_HPP_

#include <cstdio>
#include <string>

#include "merlin_hashtable.hpp"

namespace nv {
namespace merlin {

template <class K, class V, class S>
class LocalKVFile : public BaseKVFile<K, V, S> {
 public:
  LocalKVFile() : keys_fp_(nullptr), values_fp_(nullptr), scores_fp_(nullptr) {}
  ~LocalKVFile() { close(); }

  /* mode as for fopen; returns true when all three files opened */
  bool open(const std::string& keys_path, const std::string& values_path,
            const std::string& scores_path, const char* mode) {
    close();
    keys_fp_ = std::fopen(keys_path.c_str(), mode);
    values_fp_ = std::fopen(values_path.c_str(), mode);
    scores_fp_ = std::fopen(scores_path.c_str(), mode);
    if (!keys_fp_ || !values_fp_ || !scores_fp_) {
      close();
      return false;
    }
    return true;
  }

  void close() noexcept {
    if (keys_fp_) std::fclose(keys_fp_);
    if (values_fp_) std::fclose(values_fp_);
    if (scores_fp_) std::fclose(scores_fp_);
    keys_fp_ = values_fp_ = scores_fp_ = nullptr;
  }

  size_t read(const size_t n, const size_t dim, K* keys, V* vectors, S* scores) override {
    const size_t nk = std::fread(keys, sizeof(K), n, keys_fp_);
    const size_t nv = std::fread(vectors, sizeof(V) * dim, nk, values_fp_);
    const size_t ns = std::fread(scores, sizeof(S), nk, scores_fp_);
    return (nv == nk && ns == nk) ? nk : 0;
  }

  size_t write(const size_t n, const size_t dim, const K* keys, const V* vectors,
               const S* scores) override {
    const size_t nk = std::fwrite(keys, sizeof(K), n, keys_fp_);
    const size_t nv = std::fwrite(vectors, sizeof(V) * dim, n, values_fp_);
    const size_t ns = std::fwrite(scores, sizeof(S), n, scores_fp_);
    return (nk == n && nv == n && ns == n) ? n : 0;
  }

 private:
  FILE* keys_fp_;
  FILE* values_fp_;
  FILE* scores_fp_;
};

}  // namespace merlin
}  // namespace nv
#endif
