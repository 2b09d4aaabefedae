// Host-only checks of the plan API on top of fake_hip_layer.cpp (no GPU):
//   race N   - N times: plan a tensor whose plan owns index tables, let two threads call cuttExecute
//              on the handle in a loop while the main thread destroys it.  Every call must return
//              CUTT_SUCCESS or CUTT_INVALID_PLAN, and a sanitizer must stay silent (the plan may be
//              freed only after the last launch that uses it has been issued).
//   noalloc  - cuttExecuteNoAlloc with the Packed and the PackedSplit method forced: the layer's counters of
//              device allocations and table uploads must not move, and the index tables the call builds in the
//              static scratch memory must equal those cuttPlan uploads for the same tensor.
//   plans    - prints what cuttPlan chooses for a fixed list of tensors (the test compares the
//              output for a device that reports its properties with one that reports zeros).
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <thread>
#include <vector>

#include "cutt.h"
#include "cutt_ext.h"

static int race(int rounds) {
  int dim[3] = {30, 40, 50}, perm[3] = {2, 1, 0};
  std::vector<char> in(64), out(64);
  cuttSetMethodOverride(CUTT_METHOD_PACKED);
  std::atomic<int> bad{0};
  long executed = 0;
  for (int r = 0; r < rounds; r++) {
    cuttHandle h;
    if (cuttPlan(&h, 3, dim, perm, r % 2 ? 4 : 8, 0) != CUTT_SUCCESS) return 1;
    std::atomic<long> done{0};
    auto loop = [&]() {
      for (;;) {
        const cuttResult rc = cuttExecute(h, in.data(), out.data());
        if (rc == CUTT_INVALID_PLAN) return;
        if (rc != CUTT_SUCCESS) { bad++; return; }
        done++;
      }
    };
    std::thread a(loop), b(loop);
    while (done < 4) std::this_thread::yield();
    if (cuttDestroy(h) != CUTT_SUCCESS) bad++;
    a.join();
    b.join();
    executed += done;
    if (cuttDestroy(h) != CUTT_INVALID_PLAN) bad++;
  }
  std::printf("race done, rounds %d, launches %ld, unexpected results %d\n", rounds, executed, (int)bad);
  return bad ? 1 : 0;
}

extern "C" size_t fakeLastPackedTables(uint32_t* out, size_t capacity);  // fake_hip_layer.cpp

static int noalloc() {
  struct Case { std::vector<int> dim, perm; int es, method; };
  const Case cases[] = {
      {{5, 7, 11, 13, 17}, {4, 2, 0, 1, 3}, 4, CUTT_METHOD_PACKED},   {{12, 9, 31, 40}, {2, 0, 3, 1}, 8, CUTT_METHOD_PACKED},
      {{20000, 2, 50}, {2, 1, 0}, 8, CUTT_METHOD_PACKEDSPLIT},        {{331, 7, 257, 3}, {2, 1, 0, 3}, 4, CUTT_METHOD_PACKEDSPLIT},
      {{6, 5, 9, 31}, {2, 0, 3, 1}, 4, CUTT_METHOD_PACKED},           {{300, 7, 290}, {2, 1, 0}, 8, CUTT_METHOD_TILED},
  };
  std::vector<char> in(64), out(64);
  int bad = 0;
  for (const Case& c : cases) {
    std::vector<int> d = c.dim, p = c.perm;
    cuttSetMethodOverride(c.method);
    unsigned long long m0, u0, m1, u1;
    cuttDeviceCallCounts(&m0, &u0);
    if (cuttExecuteNoAlloc((int)d.size(), d.data(), p.data(), (size_t)c.es, 0, in.data(), out.data()) != CUTT_SUCCESS) return 1;
    cuttDeviceCallCounts(&m1, &u1);
    if (m1 != m0 || u1 != u0) {
      std::printf("cuttExecuteNoAlloc allocated %llu times, uploaded %llu times\n", m1 - m0, u1 - u0);
      bad++;
    }
    if (c.method == CUTT_METHOD_TILED) continue;  // no tables
    std::vector<uint32_t> built(1 << 20), uploaded(1 << 20);
    const size_t nBuilt = fakeLastPackedTables(built.data(), built.size());
    cuttHandle h;
    if (cuttPlan(&h, (int)d.size(), d.data(), p.data(), (size_t)c.es, 0) != CUTT_SUCCESS) return 1;
    cuttPlanInfo info;
    if (cuttGetPlanInfo(h, &info) != CUTT_SUCCESS || info.method != c.method) return 1;
    cuttDeviceCallCounts(&m0, &u0);
    if (m0 != m1 + 1 || u0 != u1 + 1) bad++;  // cuttPlan does allocate and upload: the counters work
    if (cuttExecute(h, in.data(), out.data()) != CUTT_SUCCESS) return 1;
    const size_t nUploaded = fakeLastPackedTables(uploaded.data(), uploaded.size());
    cuttDestroy(h);
    if (nBuilt == 0 || nBuilt != nUploaded || std::memcmp(built.data(), uploaded.data(), nBuilt * sizeof(uint32_t)) != 0) {
      std::printf("tables differ: %zu entries built in place, %zu uploaded\n", nBuilt, nUploaded);
      bad++;
    }
    std::printf("method %d: %zu table entries equal, no allocation\n", c.method, nBuilt);
  }
  cuttSetMethodOverride(0);
  std::printf("noalloc done, failures %d\n", bad);
  return bad ? 1 : 0;
}

static int plans() {
  struct Case { std::vector<int> dim, perm; int es; };
  const Case cases[] = {
      {{1024, 64, 1024, 3}, {2, 1, 0, 3}, 8}, {{5, 7, 11, 13, 17, 1093}, {4, 2, 0, 5, 1, 3}, 4},
      {{200000, 2, 500}, {2, 1, 0}, 8},       {{8192, 8192}, {1, 0}, 4},
      {{1305, 599, 88}, {0, 2, 1}, 8},        {{5, 42, 75, 86, 57}, {1, 3, 4, 2, 0}, 4},
      {{36, 3, 3, 11, 51, 4, 275}, {6, 5, 2, 4, 1, 0, 3}, 4}, {{43, 67}, {1, 0}, 8},
  };
  for (const Case& c : cases) {
    cuttHandle h;
    std::vector<int> d = c.dim, p = c.perm;
    if (cuttPlan(&h, (int)d.size(), d.data(), p.data(), (size_t)c.es, 0) != CUTT_SUCCESS) return 1;
    cuttPlanInfo i;
    if (cuttGetPlanInfo(h, &i) != CUTT_SUCCESS) return 1;
    std::printf("method %d numMm %d numMk %d split %d/%d x %d/%d blocks %lld threads %d lds %llu policy %d predicted %.3f\n",
                i.method, i.numMm, i.numMk, i.splitRank, i.numSplit, i.splitRank2, i.numSplit2, i.numBlocks,
                i.numThreads, i.ldsBytes, i.cachePolicy, i.usPredicted);
    if (!(i.usPredicted > 0.0 && i.usPredicted < 1e9)) return 1;  // a finite estimate
    cuttDestroy(h);
  }
  return 0;
}

int main(int argc, char** argv) {
  if (argc > 2 && !std::strcmp(argv[1], "race")) return race(std::atoi(argv[2]));
  if (argc > 1 && !std::strcmp(argv[1], "plans")) return plans();
  if (argc > 1 && !std::strcmp(argv[1], "noalloc")) return noalloc();
  std::printf("usage: plan_lifetime_stress race N | plans | noalloc\n");
  return 2;
}
