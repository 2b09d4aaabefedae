// Host-side stress of the planner for the sanitizer tests: four caller threads put random
// problems (ranks 2-7, both element sizes, every fourth one with power-of-two extents) through the candidate API, which enumerates the
// candidates, builds their index tables and runs the cost model on the planner's own helper
// threads.  Needs no GPU.  Prints "done, refused N".
#include <cmath>
#include <cstdio>
#include <random>
#include <thread>
#include <vector>

#include "cutt.h"
#include "cutt_ext.h"

static int work(unsigned seed, int count) {
  std::mt19937 rng(seed);
  int refused = 0;
  for (int it = 0; it < count; it++) {
    const int rank = 2 + (int)(rng() % 6);
    std::vector<int> dim(rank), perm(rank);
    const double volume = 1e5 * (1 + rng() % 2000);
    const double mean = std::pow(volume, 1.0 / rank);
    for (int r = 0; r < rank; r++) {
      dim[r] = 2 + (int)(rng() % (unsigned)(2 * mean));
      perm[r] = r;
    }
    if (it % 4 == 3) {
      // every fourth problem: extents that are powers of two, 2^26-2^28 elements - the tensors on which the
      // planner numbers workgroups and work items by address bits
      int bits = 26 + (int)(rng() % 3);
      for (int r = 0; r < rank; r++) dim[r] = 2;
      for (bits -= rank; bits > 0; bits--) dim[rng() % (unsigned)rank] *= 2;
    }
    for (int r = rank - 1; r > 0; r--) std::swap(perm[r], perm[rng() % (unsigned)(r + 1)]);
    void* list = cuttCandidatesCreate(rank, dim.data(), perm.data(), (rng() & 1) ? 4 : 8);
    if (!list) {
      refused++;
      continue;
    }
    const int n = cuttCandidatesCount(list), best = cuttCandidatesBest(list);
    cuttPlanInfo info;
    if (n < 1 || best < 0 || best >= n || cuttCandidatesInfo(list, best, &info) != 0) refused++;
    cuttCandidatesFree(list);
  }
  return refused;
}

int main(int argc, char** argv) {
  const int perThread = argc > 1 ? std::atoi(argv[1]) : 40;
  std::vector<int> refused(4, 0);
  std::vector<std::thread> threads;
  for (int i = 0; i < 4; i++) threads.emplace_back([&refused, i, perThread] { refused[i] = work(100u + i, perThread); });
  for (std::thread& t : threads) t.join();
  int total = 0;
  for (int r : refused) total += r;
  std::printf("done, refused %d\n", total);
  return 0;
}
