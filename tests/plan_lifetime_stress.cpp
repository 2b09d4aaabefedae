// Host-only checks of the plan API on top of fake_hip_layer.cpp (no GPU):
//   race N   - N times: plan a tensor whose plan owns index tables, let two threads call cuttExecute
//              on the handle in a loop while the main thread destroys it.  Every call must return
//              CUTT_SUCCESS or CUTT_INVALID_PLAN, and a sanitizer must stay silent (the plan may be
//              freed only after the last launch that uses it has been issued).
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
  std::printf("usage: plan_lifetime_stress race N | plans\n");
  return 2;
}
