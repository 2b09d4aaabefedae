/*
 * cutt_test - native correctness driver for libcutt.so on an MI355X.
 *
 * Counterpart of the reference's test program (src/cutt_test.cpp:63-484): the
 * same five groups of cases, run through the public plan API only
 * (cuttPlan / cuttPlanMeasure / cuttExecute / cuttDestroy) and verified on the
 * device against the closed form (tensor_check.h):
 *   1  every permutation of ranks 2-7 on small tensors, 4- and 8-byte elements
 *      (reference test1, :138-158)
 *   2  ranks 2-15, random volume, extents and permutation, seeded
 *      (reference test2, :164-240, which seeds from the clock)
 *   3  hand-picked shapes (reference test3, :245-366)
 *   4  ten plans on ten streams (reference test4, :371-404)
 *   5  the cost model's transaction counters against brute force
 *      (reference test5, :410-431)
 *   6  what the API refuses, and that the checker notices a wrong element
 *   7  four host threads that plan, execute, check and destroy at the same time
 *      (the reference keeps its plans in an unguarded table, src/cutt.cpp:35-39; this
 *      library guards its own)
 * Prints "test OK" or "test FAIL"; the exit status says the same.
 */
#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <set>
#include <string>
#include <thread>

#include "cutt_ext.h"
#include "driver_util.h"
#include "tensor_check.h"

using namespace cuttdrv;

namespace {

const long long kDataElems = 200LL * 1000 * 1000;  // 8-byte elements per buffer (reference src/cutt_test.cpp:52)

void* dataIn = nullptr;
void* dataOut = nullptr;
TensorChecker* checker = nullptr;
BwStats* stats4 = nullptr;
BwStats* stats8 = nullptr;
bool useMeasure = false;
bool verbose = false;
long long numTensors = 0;

// Every transpose in this file goes through this guard before it touches the buffers.
bool fitsBuffers(const std::vector<int>& dim, size_t elemSize) {
  long long vol = volumeOf(dim);
  if (vol * (long long)elemSize <= kDataElems * 8) return true;
  std::printf("tensor of %lld elements of %zu bytes does not fit the buffers\n", vol, elemSize);
  return false;
}

bool testTensor(std::vector<int> dim, std::vector<int> perm, size_t elemSize) {
  int rank = (int)dim.size();
  long long vol = volumeOf(dim);
  if (!fitsBuffers(dim, elemSize)) return false;
  if (verbose) {
    std::printf("elements %lld elemsize %zu\n", vol, elemSize);
    printVec("  dimensions ", dim);
    printVec("  permutation", perm);
  }
  BwStats* st = elemSize == 4 ? stats4 : stats8;
  cuttHandle plan;
  if (useMeasure)
    CUTT_CHECK(cuttPlanMeasure(&plan, rank, dim.data(), perm.data(), elemSize, 0, dataIn, dataOut));
  else
    CUTT_CHECK(cuttPlan(&plan, rank, dim.data(), perm.data(), elemSize, 0));
  checker->fillBytes(dataOut, 0xff, (size_t)vol * elemSize);
  HIP_CHECK(hipDeviceSynchronize());
  bool timed = vol > 1000000;
  if (timed) st->start(0);
  CUTT_CHECK(cuttExecute(plan, dataIn, dataOut));
  if (timed) {
    st->stop(0);
    st->record(dim, perm);
  }
  HIP_CHECK(hipDeviceSynchronize());
  bool ok = checker->checkAndReport(rank, dim.data(), perm.data(), elemSize, dataOut);
  if (!ok) {
    cuttPlanInfo info;
    if (cuttGetPlanInfo(plan, &info) == CUTT_SUCCESS)
      std::printf("  plan: method %d numMm %d numMk %d numSplit %d/%d blocks %lld threads %d\n", info.method, info.numMm,
                  info.numMk, info.numSplit, info.numSplit2, info.numBlocks, info.numThreads);
    std::printf("  elemsize %zu\n", elemSize);
    printVec("  dimensions ", dim);
    printVec("  permutation", perm);
  }
  CUTT_CHECK(cuttDestroy(plan));
  numTensors++;
  return ok;
}

bool testBoth(const std::vector<int>& dim, const std::vector<int>& perm) {
  return testTensor(dim, perm, 8) && testTensor(dim, perm, 4);
}

bool test1() {
  const int minDim = 2, maxDim = 16;
  for (int rank = 2; rank <= 7; rank++) {
    std::vector<int> dim(rank), perm(rank);
    for (int r = 0; r < rank; r++) {
      perm[r] = r;
      dim[r] = minDim + r * (maxDim - minDim) / rank;
    }
    do {
      if (!testBoth(dim, perm)) return false;
    } while (std::next_permutation(perm.begin(), perm.end()));
    std::printf("test1: rank %d done\n", rank);
    std::fflush(stdout);
  }
  return true;
}

bool test2(uint64_t seed, int samples) {
  Rng rng(seed);
  for (int rank = 2; rank <= 15; rank++) {
    double volMin = std::pow(3.0, rank), volMax = (double)kDataElems;
    for (int s = 0; s < samples; s++) {
      std::vector<int> dim, perm(rank);
      for (int r = 0; r < rank; r++) perm[r] = r;
      bool found = false;
      for (int tries = 0; tries < 100 && !found; tries++) {
        double vol = volMin + (volMax - volMin) * rng.uniform();
        found = randomDims(rng, vol, rank, 0.3, dim) && (double)volumeOf(dim) <= volMax;
      }
      if (!found) {
        std::printf("test2: no extents found for rank %d\n", rank);
        return false;
      }
      rng.shuffle(perm);
      if (!testBoth(dim, perm)) return false;
    }
    std::printf("test2: rank %d done\n", rank);
    std::fflush(stdout);
  }
  return true;
}

// Tensors that one launch cannot address are transposed piece by piece (tensors of 2^32 elements and
// more in production).  CUTT_SPAN_LIMIT lowers the limit, so that random tensors of ordinary size
// take that path here: both planners, both element sizes, checked like every other tensor.  The
// reference has no counterpart (its volumes are ints).
bool test8(uint64_t seed, int samples) {
  Rng rng(seed + 8);
  int cut = 0;
  for (int rank = 2; rank <= 8; rank++) {
    for (int s = 0; s < std::max(1, samples / 5); s++) {
      std::vector<int> dim, perm(rank);
      for (int r = 0; r < rank; r++) perm[r] = r;
      bool found = false;
      for (int tries = 0; tries < 100 && !found; tries++) {
        double vol = 2e5 + 2e7 * rng.uniform();
        found = randomDims(rng, vol, rank, 0.3, dim);
      }
      if (!found) return false;
      rng.shuffle(perm);
      const long long vol = volumeOf(dim);
      const long long limit = vol / 9 + (long long)((double)vol * 0.4 * rng.uniform());
      setenv("CUTT_SPAN_LIMIT", std::to_string(limit).c_str(), 1);
      // shapes that cannot be cut (the fastest rank of one side fixed on the other) are refused; skip them
      cuttHandle probe;
      cuttResult rc = cuttPlan(&probe, rank, dim.data(), perm.data(), 4, 0);
      bool ok = true;
      if (rc == CUTT_SUCCESS) {
        cuttPlanInfo info;
        CUTT_CHECK(cuttGetPlanInfo(probe, &info));
        CUTT_CHECK(cuttDestroy(probe));
        if (info.numPieces > 1) cut++;
        ok = testBoth(dim, perm);
      } else if (rc != CUTT_INVALID_PARAMETER) {
        ok = false;
      }
      unsetenv("CUTT_SPAN_LIMIT");
      if (!ok) return false;
    }
  }
  std::printf("test8: %d tensors went in pieces\n", cut);
  return cut > 0;
}

bool test3() {
  struct Case {
    std::vector<int> dim, perm;
  };
  const Case cases[] = {
      {{43, 67}, {1, 0}},
      {{65536 * 32, 2}, {1, 0}},
      {{1305, 599, 88}, {0, 2, 1}},
      {{24, 330, 64, 147}, {1, 0, 2, 3}},
      {{2, 5, 9, 12}, {0, 1, 2, 3}},
      {{2, 4, 6, 9, 11, 13}, {0, 1, 2, 3, 4, 5}},
      {{5, 42, 75, 86, 57}, {1, 3, 4, 2, 0}},
      {{5, 3, 2, 9, 14}, {0, 1, 3, 2, 4}},
  };
  for (const Case& c : cases)
    if (!testBoth(c.dim, c.perm)) return false;
  return true;
}

bool test4() {
  std::vector<int> dim = {24, 32, 16, 36, 43, 9};
  std::vector<int> perm = {5, 1, 4, 2, 3, 0};
  if (!fitsBuffers(dim, 8)) return false;
  const int numStream = 10;
  hipStream_t streams[numStream];
  cuttHandle plans[numStream];
  for (int i = 0; i < numStream; i++) HIP_CHECK(hipStreamCreate(&streams[i]));
  HIP_CHECK(hipDeviceSynchronize());
  for (int i = 0; i < numStream; i++) {
    CUTT_CHECK(cuttPlan(&plans[i], (int)dim.size(), dim.data(), perm.data(), 8, streams[i]));
    CUTT_CHECK(cuttExecute(plans[i], dataIn, dataOut));
  }
  HIP_CHECK(hipDeviceSynchronize());
  bool ok = checker->checkAndReport((int)dim.size(), dim.data(), perm.data(), 8, dataOut);
  for (int i = 0; i < numStream; i++) {
    CUTT_CHECK(cuttDestroy(plans[i]));
    HIP_CHECK(hipStreamDestroy(streams[i]));
  }
  return ok;
}

// Counters against brute force, at the widths the model uses on gfx950: 128-byte lines and
// 32-byte sectors of 8- and 4-byte elements, 64-lane requests.
bool test5(uint64_t seed) {
  Rng rng(seed ^ 0x5555);
  const int widths[][2] = {{16, 4}, {32, 8}, {16, 16}, {32, 32}};
  for (int iter = 0; iter < 4000; iter++) {
    int acc = widths[iter % 4][0], cache = widths[iter % 4][1];
    int n = 1 + rng.below(64);
    std::set<int> posSet;
    bool contiguous = (iter & 4) != 0;
    int start = rng.below(500);
    if (contiguous) {
      for (int i = 0; i < n; i++) posSet.insert(start + i);
    } else {
      for (int i = 0; i < n; i++) posSet.insert(rng.below(600));
    }
    std::vector<int> pos(posSet.begin(), posSet.end());
    n = (int)pos.size();
    // brute force
    std::set<int> lines;
    std::map<int, int> sectors;
    for (int p : pos) {
      lines.insert(p / acc);
      sectors[p / cache]++;
    }
    int full = 0, part = 0;
    for (auto& kv : sectors) (kv.second == cache ? full : part)++;
    // library
    std::vector<int> segAcc(n), segCache(n);
    for (int i = 0; i < n; i++) {
      segAcc[i] = pos[i] / acc;
      segCache[i] = pos[i] / cache;
    }
    int tran = cuttModelGlTransactionsSeg(segAcc.data(), n);
    int f = 0, p = 0;
    cuttModelCacheLinesSeg(segCache.data(), n, cache, &f, &p);
    if (tran != (int)lines.size() || f != full || p != part) {
      std::printf("test5: scattered counters differ: tran %d/%zu full %d/%d part %d/%d (acc %d cache %d n %d)\n", tran,
                  lines.size(), f, full, p, part, acc, cache, n);
      return false;
    }
    if (contiguous) {
      int tranC = cuttModelGlTransactionsCont(start, n, acc);
      int fc = 0, pc = 0;
      cuttModelCacheLinesCont(start, n, cache, &fc, &pc);
      if (tranC != tran || fc != full || pc != part) {
        std::printf("test5: contiguous counters differ at pos %d n %d acc %d cache %d\n", start, n, acc, cache);
        return false;
      }
    }
  }
  // LDS bank conflicts: strides of a gather (c, d, ct per rank) replayed lane by lane
  for (int iter = 0; iter < 300; iter++) {
    int nRank = 1 + rng.below(3);
    std::vector<int> msh;
    int vol = 1, c = 1;
    std::vector<int> ext(nRank);
    for (int r = 0; r < nRank; r++) {
      ext[r] = 2 + rng.below(12);
      vol *= ext[r];
    }
    std::vector<int> order(nRank);
    for (int r = 0; r < nRank; r++) order[r] = r;
    rng.shuffle(order);
    // ct: stride of rank r in a tensor whose ranks are laid out in `order`
    std::vector<int> ct(nRank);
    int acc = 1;
    for (int k = 0; k < nRank; k++) {
      ct[order[k]] = acc;
      acc *= ext[order[k]];
    }
    for (int r = 0; r < nRank; r++) {
      msh.push_back(c);
      msh.push_back(ext[r]);
      msh.push_back(ct[r]);
      c *= ext[r];
    }
    int numThreads = 64 * (1 + rng.below(4));
    const int wave = 64, banks = 64;
    int ld = 0, req = 0;
    for (int b0 = 0; b0 < vol; b0 += numThreads)
      for (int w0 = b0; w0 < std::min(vol, b0 + numThreads); w0 += wave) {
        std::map<int, int> cnt;
        int worst = 0;
        for (int j = w0; j < std::min(w0 + wave, vol); j++) {
          int p = 0;
          for (int r = 0; r < nRank; r++) p += ((j / msh[3 * r]) % msh[3 * r + 1]) * msh[3 * r + 2];
          worst = std::max(worst, ++cnt[p % banks]);
        }
        ld += worst;
        req++;
      }
    int out4[4];
    cuttModelShTransactions(wave, banks, numThreads, vol, msh.data(), nRank, out4);
    if (out4[0] != ld || out4[1] != req || out4[2] != req || out4[3] != req) {
      std::printf("test5: LDS counters differ: %d %d %d %d, brute force %d %d\n", out4[0], out4[1], out4[2], out4[3], ld, req);
      return false;
    }
  }
  return true;
}

#define EXPECT(cond)                                              \
  do {                                                            \
    if (!(cond)) {                                                \
      std::printf("test6: expectation failed: %s\n", #cond);      \
      return false;                                               \
    }                                                             \
  } while (0)

bool test6() {
  int dim[3] = {31, 17, 45}, perm[3] = {2, 0, 1};
  if (!fitsBuffers({31, 17, 45}, 4)) return false;
  cuttHandle h = 0;
  // what cuttPlan refuses (reference src/cutt.cpp:59-82)
  int bad2[3] = {2, 0, 0}, bad3[3] = {3, 0, 1}, one[3] = {31, 1, 45};
  EXPECT(cuttPlan(&h, 3, dim, perm, 2, 0) == CUTT_INVALID_PARAMETER);
  EXPECT(cuttPlan(&h, 1, dim, perm, 4, 0) == CUTT_INVALID_PARAMETER);
  EXPECT(cuttPlan(&h, 3, dim, bad2, 4, 0) == CUTT_INVALID_PARAMETER);
  EXPECT(cuttPlan(&h, 3, dim, bad3, 4, 0) == CUTT_INVALID_PARAMETER);
  EXPECT(cuttPlan(&h, 3, one, perm, 4, 0) == CUTT_INVALID_PARAMETER);
  EXPECT(cuttPlanMeasure(&h, 3, dim, perm, 4, 0, dataIn, dataIn) == CUTT_INVALID_PARAMETER);
  // what cuttExecute and cuttDestroy refuse (reference src/cutt.cpp:286-310)
  EXPECT(cuttPlan(&h, 3, dim, perm, 4, 0) == CUTT_SUCCESS);
  EXPECT(cuttExecute(h, dataIn, dataIn) == CUTT_INVALID_PARAMETER);
  EXPECT(cuttExecute(h + 12345, dataIn, dataOut) == CUTT_INVALID_PLAN);
  EXPECT(cuttExecute(h, dataIn, dataOut) == CUTT_SUCCESS);
  HIP_CHECK(hipDeviceSynchronize());
  EXPECT(checker->check(3, dim, perm, 4, dataOut).numWrong == 0);
  // the checker must notice one wrong element and name it
  unsigned int wrong = 0xdeadbeef;
  const unsigned long long at = 4242;
  HIP_CHECK(hipMemcpy((char*)dataOut + at * 4, &wrong, 4, hipMemcpyHostToDevice));
  CheckResult r = checker->check(3, dim, perm, 4, dataOut);
  EXPECT(r.numWrong == 1 && r.firstPos == at && r.got == wrong);
  // and a transposed operand: checking against the inverse permutation must fail
  int inv[3] = {1, 2, 0};
  EXPECT(cuttExecute(h, dataIn, dataOut) == CUTT_SUCCESS);
  HIP_CHECK(hipDeviceSynchronize());
  EXPECT(checker->check(3, dim, inv, 4, dataOut).numWrong > 0);
  EXPECT(cuttDestroy(h) == CUTT_SUCCESS);
  EXPECT(cuttDestroy(h) == CUTT_INVALID_PLAN);
  EXPECT(cuttExecute(h, dataIn, dataOut) == CUTT_INVALID_PLAN);
  return true;
}

// Four host threads, each with a stream, a checker and a quarter of the output buffer of its own,
// plan (every third tensor with cuttPlanMeasure), execute, check and destroy seeded random tensors
// at the same time.  The input buffer is shared and only read.
bool test7(uint64_t seed) {
  const int numThreads = 4, tensorsPerThread = 12;
  const size_t sliceBytes = (size_t)kDataElems * 8 / numThreads;
  std::atomic<int> failures{0};
  std::atomic<long long> done{0};
  std::mutex printMutex;
  auto fail = [&](int t, const char* what, const std::vector<int>& dim, const std::vector<int>& perm, size_t es) {
    std::lock_guard<std::mutex> lock(printMutex);
    std::printf("test7: thread %d: %s, elemsize %zu\n", t, what, es);
    printVec("  dimensions ", dim);
    printVec("  permutation", perm);
    failures++;
  };
  auto worker = [&](int t) {
    Rng rng(seed * 7919 + (uint64_t)t);
    TensorChecker mine;
    hipStream_t stream;
    if (hipStreamCreate(&stream) != hipSuccess) {
      failures++;
      return;
    }
    char* out = (char*)dataOut + (size_t)t * sliceBytes;
    for (int i = 0; i < tensorsPerThread && failures == 0; i++) {
      const int rank = 2 + rng.below(6);
      const size_t es = (i + t) % 2 ? 4 : 8;
      std::vector<int> dim, perm(rank);
      for (int r = 0; r < rank; r++) perm[r] = r;
      const double vol = std::max(std::pow(3.0, rank), 1e4 + 4e6 * rng.uniform());
      if (!randomDims(rng, vol, rank, 0.3, dim) || (size_t)volumeOf(dim) * es > sliceBytes) continue;
      rng.shuffle(perm);
      cuttHandle plan = 0;
      cuttResult r = i % 3 == 2 ? cuttPlanMeasure(&plan, rank, dim.data(), perm.data(), es, stream, dataIn, out)
                                : cuttPlan(&plan, rank, dim.data(), perm.data(), es, stream);
      if (r != CUTT_SUCCESS) {
        fail(t, "plan refused", dim, perm, es);
        break;
      }
      bool ok = hipMemsetAsync(out, 0xff, (size_t)volumeOf(dim) * es, stream) == hipSuccess;
      ok = ok && cuttExecute(plan, dataIn, out) == CUTT_SUCCESS;
      ok = ok && hipStreamSynchronize(stream) == hipSuccess;
      if (!ok) fail(t, "execute failed", dim, perm, es);
      else if (mine.check(rank, dim.data(), perm.data(), es, out).numWrong != 0) fail(t, "wrong result", dim, perm, es);
      if (cuttDestroy(plan) != CUTT_SUCCESS) fail(t, "destroy refused", dim, perm, es);
      done++;
    }
    (void)hipStreamDestroy(stream);
  };
  HIP_CHECK(hipDeviceSynchronize());
  std::vector<std::thread> threads;
  for (int t = 0; t < numThreads; t++) threads.emplace_back(worker, t);
  for (std::thread& th : threads) th.join();
  HIP_CHECK(hipDeviceSynchronize());
  numTensors += done;
  return failures == 0 && done > 0;
}

void usage() {
  std::printf("cutt_test [options]\n");
  std::printf("Options:\n");
  std::printf("-device gpuid   : use GPU with ID gpuid\n");
  std::printf("-seed n         : seed of the random cases (default 1)\n");
  std::printf("-samples n      : random tensors per rank in test 2 (default 100)\n");
  std::printf("-tests list     : comma-separated tests to run, e.g. 1,3,4 (default all)\n");
  std::printf("-measure        : plan with cuttPlanMeasure instead of cuttPlan\n");
  std::printf("-verbose        : print every tensor\n");
}

}  // namespace

int main(int argc, char* argv[]) {
  int gpuid = -1, samples = 100;
  uint64_t seed = 1;
  std::set<int> tests = {1, 2, 3, 4, 5, 6, 7, 8};
  for (int i = 1; i < argc; i++) {
    std::string a = argv[i];
    if (a == "-device" && i + 1 < argc) {
      gpuid = std::atoi(argv[++i]);
    } else if (a == "-seed" && i + 1 < argc) {
      seed = std::strtoull(argv[++i], nullptr, 10);
    } else if (a == "-samples" && i + 1 < argc) {
      samples = std::atoi(argv[++i]);
    } else if (a == "-tests" && i + 1 < argc) {
      tests.clear();
      for (char* tok = std::strtok(argv[++i], ","); tok; tok = std::strtok(nullptr, ",")) tests.insert(std::atoi(tok));
    } else if (a == "-measure") {
      useMeasure = true;
    } else if (a == "-verbose") {
      verbose = true;
    } else {
      usage();
      return 1;
    }
  }
  if (gpuid >= 0) HIP_CHECK(hipSetDevice(gpuid));

  stats4 = new BwStats(4);
  stats8 = new BwStats(8);
  HIP_CHECK(hipMalloc(&dataIn, (size_t)kDataElems * 8));
  HIP_CHECK(hipMalloc(&dataOut, (size_t)kDataElems * 8));
  checker = new TensorChecker();
  checker->fillPattern(dataIn, (size_t)kDataElems * 2);

  bool ok = true;
  struct Entry {
    int id;
    const char* what;
  };
  const Entry entries[] = {{1, "all permutations, ranks 2-7"}, {2, "random tensors, ranks 2-15"}, {3, "hand-picked shapes"},
                           {4, "ten streams"},                 {5, "model counters"},             {6, "refusals and checker"},
                           {7, "four host threads"},           {8, "tensors cut into pieces"}};
  for (const Entry& e : entries) {
    if (!ok || !tests.count(e.id)) continue;
    std::printf("test %d: %s\n", e.id, e.what);
    std::fflush(stdout);
    switch (e.id) {
      case 1: ok = test1(); break;
      case 2: ok = test2(seed, samples); break;
      case 3: ok = test3(); break;
      case 4: ok = test4(); break;
      case 5: ok = test5(seed); break;
      case 6: ok = test6(); break;
      case 7: ok = test7(seed); break;
      case 8: ok = test8(seed, samples); break;
    }
    std::printf("test %d %s\n", e.id, ok ? "passed" : "FAILED");
    std::fflush(stdout);
  }

  if (ok) {
    for (BwStats* st : {stats8, stats4}) {
      const BwSample* w = st->worst();
      if (!w) continue;
      std::printf("worst bandwidth over tensors above 1M elements, %d-byte elements: %4.2f GB/s\n", st == stats8 ? 8 : 4, w->gbs);
      printVec("  dimensions ", w->dim);
      printVec("  permutation", w->perm);
    }
  }
  std::printf("tensors transposed and checked: %lld, seed %llu\n", numTensors, (unsigned long long)seed);
  std::printf(ok ? "test OK\n" : "test FAIL\n");

  delete checker;
  HIP_CHECK(hipFree(dataIn));
  HIP_CHECK(hipFree(dataOut));
  delete stats4;
  delete stats8;
  return ok ? 0 : 1;
}
