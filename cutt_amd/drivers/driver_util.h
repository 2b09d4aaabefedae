/*
 * driver_util.h - what the native test and benchmark drivers share: error
 * checks, a seeded generator, tensor-shape generators and bandwidth
 * statistics per rank.
 *
 * The statistics follow the reference's cuttTimer (src/cuttTimer.h:66-121,
 * src/cuttTimer.cpp:89-246): bandwidth = 2 * volume * sizeof(element) / time in
 * GB/s (1e9 bytes), grouped by tensor rank, with best / worst / average /
 * median and the worst case's shape.  Times come from HIP events on the
 * plan's stream.
 */
#ifndef CUTT_DRIVERS_UTIL_H
#define CUTT_DRIVERS_UTIL_H

#include <hip/hip_runtime_api.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <map>
#include <vector>

#include "cutt.h"

#define HIP_CHECK(call)                                                                     \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      std::fprintf(stderr, "%s:%d HIP error %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
      std::exit(2);                                                                         \
    }                                                                                       \
  } while (0)

#define CUTT_CHECK(call)                                                                 \
  do {                                                                                   \
    cuttResult r_ = (call);                                                              \
    if (r_ != CUTT_SUCCESS) {                                                            \
      std::fprintf(stderr, "%s:%d cutt error %d in %s\n", __FILE__, __LINE__, (int)r_, #call); \
      std::exit(2);                                                                      \
    }                                                                                    \
  } while (0)

namespace cuttdrv {

// splitmix64: the same sequence on every platform, unlike std:: distributions.
class Rng {
 public:
  explicit Rng(uint64_t seed) : s_(seed) {}
  uint64_t next() {
    uint64_t z = (s_ += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
  }
  double uniform() { return (double)(next() >> 11) * (1.0 / 9007199254740992.0); }  // [0, 1)
  int below(int n) { return (int)(uniform() * n); }
  double normal(double mean, double sigma) {
    double u1 = 1.0 - uniform(), u2 = uniform();
    return mean + sigma * std::sqrt(-2.0 * std::log(u1)) * std::cos(6.283185307179586 * u2);
  }
  template <typename T>
  void shuffle(std::vector<T>& v) {
    for (int i = (int)v.size() - 1; i > 0; i--) std::swap(v[i], v[below(i + 1)]);
  }

 private:
  uint64_t s_;
};

inline bool isIdentity(const std::vector<int>& p) {
  for (size_t i = 0; i < p.size(); i++)
    if (p[i] != (int)i) return false;
  return true;
}

inline long long volumeOf(const std::vector<int>& dim) {
  long long v = 1;
  for (int d : dim) v *= d;
  return v;
}

inline void printVec(const char* label, const std::vector<int>& v) {
  std::printf("%s", label);
  for (int x : v) std::printf(" %d", x);
  std::printf("\n");
}

// Random extents (each >= 2) whose product lies within `tol` (relative) of `vol`: draw every extent
// around the geometric mean, rescale all to the wanted volume, then walk single extents up or down
// while that brings the product closer.  Returns false if it cannot get within tol.
inline bool randomDims(Rng& rng, double vol, int rank, double tol, std::vector<int>& dim) {
  dim.assign(rank, 2);
  double mean = std::floor(std::pow(vol, 1.0 / rank));
  if (mean < 2.0) return false;
  for (int attempt = 0; attempt < 2000; attempt++) {
    double cur = 1.0;
    std::vector<double> f(rank);
    for (int r = 0; r < rank; r++) {
      f[r] = std::max(1.0, mean + (2.0 * rng.uniform() - 1.0) * (mean - 2.0));
      cur *= f[r];
    }
    double scale = std::pow(vol / cur, 1.0 / rank);
    cur = 1.0;
    for (int r = 0; r < rank; r++) {
      dim[r] = std::max(2, (int)std::lround(f[r] * scale));
      cur *= dim[r];
    }
    for (int pass = 0; pass < 4 * rank && std::fabs(cur - vol) / vol > tol; pass++) {
      int r = rng.below(rank);
      int d = cur < vol ? dim[r] + 1 : std::max(2, dim[r] - 1);
      double next = cur / dim[r] * d;
      if (std::fabs(next - vol) < std::fabs(cur - vol)) {
        dim[r] = d;
        cur = next;
      }
    }
    if (std::fabs(cur - vol) / vol <= tol && cur < 2147483647.0) return true;
  }
  return false;
}

struct BwSample {
  double gbs;
  std::vector<int> dim, perm;
};

class BwStats {
 public:
  explicit BwStats(size_t elemSize) : elemSize_(elemSize) {
    HIP_CHECK(hipEventCreate(&t0_));
    HIP_CHECK(hipEventCreate(&t1_));
  }
  ~BwStats() {
    (void)hipEventDestroy(t0_);
    (void)hipEventDestroy(t1_);
  }
  BwStats(const BwStats&) = delete;
  BwStats& operator=(const BwStats&) = delete;

  void start(hipStream_t s) { HIP_CHECK(hipEventRecord(t0_, s)); }
  // Stops the clock; returns the elapsed milliseconds.
  double stop(hipStream_t s) {
    HIP_CHECK(hipEventRecord(t1_, s));
    HIP_CHECK(hipEventSynchronize(t1_));
    float ms = 0;
    HIP_CHECK(hipEventElapsedTime(&ms, t0_, t1_));
    lastMs_ = ms;
    return ms;
  }
  double lastMs() const { return lastMs_; }
  double gbs(long long vol) const { return 2.0 * (double)vol * (double)elemSize_ / (lastMs_ * 1e-3) / 1e9; }
  // Record the last interval for this tensor.
  void record(const std::vector<int>& dim, const std::vector<int>& perm) {
    byRank_[(int)dim.size()].push_back({gbs(volumeOf(dim)), dim, perm});
  }
  // Replace the entry recorded last for this rank if the new interval is faster (best of N runs).
  void recordBest(const std::vector<int>& dim, const std::vector<int>& perm, bool first) {
    if (first) {
      record(dim, perm);
      return;
    }
    BwSample& s = byRank_[(int)dim.size()].back();
    s.gbs = std::max(s.gbs, gbs(volumeOf(dim)));
  }
  bool empty() const { return byRank_.empty(); }

  void printSummary(bool withData) const {
    if (withData) {
      for (const auto& kv : byRank_) {
        std::printf("RANK%d", kv.first);
        for (const BwSample& s : kv.second) std::printf(" %1.2f", s.gbs);
        std::printf("\n");
      }
    }
    std::printf("rank samples best worst average median   (GB/s)\n");
    for (const auto& kv : byRank_) {
      std::vector<double> v;
      for (const BwSample& s : kv.second) v.push_back(s.gbs);
      std::sort(v.begin(), v.end());
      double sum = 0;
      for (double x : v) sum += x;
      double med = v.size() % 2 ? v[v.size() / 2] : 0.5 * (v[v.size() / 2 - 1] + v[v.size() / 2]);
      std::printf("%d %zu %8.2f %8.2f %8.2f %8.2f\n", kv.first, v.size(), v.back(), v.front(), sum / v.size(), med);
    }
    for (const auto& kv : byRank_) {
      const BwSample* worst = &kv.second[0];
      for (const BwSample& s : kv.second)
        if (s.gbs < worst->gbs) worst = &s;
      std::printf("rank %d worst %4.2f GB/s\n", kv.first, worst->gbs);
      printVec("  dimensions ", worst->dim);
      printVec("  permutation", worst->perm);
    }
  }
  // Worst sample over all ranks (nullptr if none).
  const BwSample* worst() const {
    const BwSample* w = nullptr;
    for (const auto& kv : byRank_)
      for (const BwSample& s : kv.second)
        if (!w || s.gbs < w->gbs) w = &s;
    return w;
  }
  std::vector<double> all() const {
    std::vector<double> v;
    for (const auto& kv : byRank_)
      for (const BwSample& s : kv.second) v.push_back(s.gbs);
    return v;
  }

 private:
  size_t elemSize_;
  hipEvent_t t0_, t1_;
  double lastMs_ = 0;
  std::map<int, std::vector<BwSample>> byRank_;
};

}  // namespace cuttdrv

#endif
