/*
 * cutt_bench - native benchmark driver for libcutt.so on an MI355X.
 *
 * Counterpart of the reference's benchmark program (src/cutt_bench.cpp:80-909)
 * with the same command line and the same suites, run through the public plan
 * API only and verified on the device after the timed runs:
 *   -dim ... -permutation ...   one tensor (reference bench_input, :440-449)
 *   -bench 3     ranks 2-8 and 15, random extents and permutation, 50 each,
 *                about 200M elements (reference bench3, :414-431)
 *   -bench 5RR   ranks 2-7, 500 random tensors each with max/min extent ratio
 *                RR, volumes normally distributed around 200M elements
 *                (reference bench5, :455-546; the README's plot protocol)
 *   -bench 6     the 57 tensors of the TTC paper's benchmark
 *                (reference bench6, :551-683)
 *   -bench 7     ranks 8 and 12 with four large and otherwise small extents
 *                (reference bench7, :688-728)
 *   -memcpy n    plain copies of n elements (reference bench_memcpy, :843-892)
 * Timing follows the reference's inner loop (:818-830): four repetitions, each
 * output fill + device synchronise + timed cuttExecute; every repetition's
 * bandwidth 2 * bytes / time enters the statistics.  A device-to-device
 * hipMemcpy of the same size is timed beside each tensor unless -nomemcpy.
 */
#include <chrono>
#include <cctype>
#include <cstring>
#include <string>

#include "cutt_ext.h"
#include "driver_util.h"
#include "tensor_check.h"

using namespace cuttdrv;

namespace {

const long long kMillion = 1000000;

void* dataIn = nullptr;
void* dataOut = nullptr;
long long dataElems = 0;  // elements of the chosen size per buffer
size_t elemSize = 8;
TensorChecker* checker = nullptr;
BwStats* stats = nullptr;
BwStats* copyStats = nullptr;
bool useMeasure = false, usePlanTimer = false, timeMemcpy = true;
int samplesOverride = 0;
std::vector<double> pctOfMemcpy;

const char* methodNames[] = {"Unknown", "Trivial", "Packed", "PackedSplit", "Tiled", "TiledCopy"};

bool benchTensor(const std::vector<int>& dimIn, const std::vector<int>& permIn) {
  std::vector<int> dim = dimIn, perm = permIn;
  int rank = (int)dim.size();
  long long vol = volumeOf(dim);
  if (vol > dataElems) {
    std::printf("benchTensor: %lld elements exceed the buffers (%lld)\n", vol, dataElems);
    return false;
  }
  std::printf("number of elements %lld\n", vol);
  printVec("dimensions ", dim);
  printVec("permutation", perm);

  cuttHandle plan;
  auto t0 = std::chrono::steady_clock::now();
  if (useMeasure)
    CUTT_CHECK(cuttPlanMeasure(&plan, rank, dim.data(), perm.data(), elemSize, 0, dataIn, dataOut));
  else
    CUTT_CHECK(cuttPlan(&plan, rank, dim.data(), perm.data(), elemSize, 0));
  double planMs = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  if (usePlanTimer) std::printf("plan took %f ms\n", planMs);
  cuttPlanInfo info;
  CUTT_CHECK(cuttGetPlanInfo(plan, &info));
  std::printf("method %s blocks %lld threads %d lds %llu candidates %d%s\n", methodNames[info.method], info.numBlocks,
              info.numThreads, info.ldsBytes, info.numCandidates, info.tiledGrouped ? " rows-in-groups" : "");
  if (info.numPieces > 1)  // a tensor beyond one launch: the line above describes the plan of the first piece
    std::printf("pieces %d shapes %d\n", info.numPieces, info.numShapes);
  // what the cost model counted for this plan, to set beside hardware counters (128-byte lines)
  std::printf("model: predicted %.1f us, lines read %.0f written %.0f partly written %.0f, LDS cycles %.0f\n", info.usPredicted,
              info.rdLines, info.wrLines, info.wrPartialLines, info.ldsCycles);

  double bestGbs = 0;
  for (int i = 0; i < 4; i++) {
    checker->fillBytes(dataOut, 0xff, (size_t)vol * elemSize);
    HIP_CHECK(hipDeviceSynchronize());
    stats->start(0);
    CUTT_CHECK(cuttExecute(plan, dataIn, dataOut));
    double ms = stats->stop(0);
    stats->record(dim, perm);
    bestGbs = std::max(bestGbs, stats->gbs(vol));
    std::printf("wall time %f ms %f GB/s\n", ms, stats->gbs(vol));
  }
  CUTT_CHECK(cuttDestroy(plan));
  bool ok = checker->checkAndReport(rank, dim.data(), perm.data(), elemSize, dataOut);

  if (ok && timeMemcpy) {
    double best = 0;
    for (int i = 0; i < 3; i++) {
      HIP_CHECK(hipDeviceSynchronize());
      copyStats->start(0);
      HIP_CHECK(hipMemcpyAsync(dataOut, dataIn, (size_t)vol * elemSize, hipMemcpyDeviceToDevice, 0));
      copyStats->stop(0);
      best = std::max(best, copyStats->gbs(vol));
    }
    pctOfMemcpy.push_back(100.0 * bestGbs / best);
    std::printf("memcpy %f GB/s, transpose at %.1f %% of it\n", best, 100.0 * bestGbs / best);
  }
  std::fflush(stdout);
  return ok;
}

bool bench3(Rng& rng, long long numElem) {
  const int ranks[] = {2, 3, 4, 5, 6, 7, 8, 15};
  int samples = samplesOverride ? samplesOverride : 50;
  for (int rank : ranks) {
    std::vector<int> dim, perm(rank);
    for (int r = 0; r < rank; r++) perm[r] = r;
    for (int s = 0; s < samples; s++) {
      rng.shuffle(perm);
      if (!randomDims(rng, (double)numElem, rank, 0.3, dim)) {
        std::printf("bench3: no extents found for rank %d\n", rank);
        return false;
      }
      if (!benchTensor(dim, perm)) return false;
    }
  }
  return true;
}

// Extents grow linearly from the smallest to `ratio` times the smallest, are scaled to the drawn
// volume, nudged to within 5 %, then shuffled.
bool bench5(Rng& rng, long long numElemAvg, int ratio) {
  int samples = samplesOverride ? samplesOverride : 500;
  if (ratio < 1) ratio = 1;
  for (int rank = 2; rank <= 7; rank++) {
    for (int iter = 0; iter < samples; iter++) {
      double numElem;
      do {
        numElem = rng.normal((double)numElemAvg, 0.2 * (double)numElemAvg);
      } while (numElem < 0.2 * (double)numElemAvg || numElem > (double)dataElems);
      std::vector<double> f(rank);
      double volf = 1.0;
      for (int r = 0; r < rank; r++) {
        f[r] = 1.0 + (double)r * (ratio - 1.0) / (double)(rank - 1);
        volf *= f[r];
      }
      double scale = std::pow(numElem / volf, 1.0 / rank);
      std::vector<int> dim(rank), perm(rank);
      double vol = 1.0;
      for (int r = 0; r < rank; r++) {
        dim[r] = std::max(2, (int)std::lround(f[r] * scale));
        if (r == rank - 1) dim[r] = std::max(2, ratio * dim[0]);
        vol *= dim[r];
        perm[r] = r;
      }
      for (int r = 1; r < rank && std::fabs(vol - numElem) / numElem > 0.05; r++) {
        int d = std::max(2, dim[r] + (vol < numElem ? 1 : -1));
        vol = vol / dim[r] * d;
        dim[r] = d;
      }
      if (vol > (double)dataElems) {
        iter--;
        continue;
      }
      rng.shuffle(dim);
      do {
        rng.shuffle(perm);
      } while (isIdentity(perm));
      if (!benchTensor(dim, perm)) return false;
    }
  }
  return true;
}

bool bench6() {
  // the 57 (extents; permutation) pairs of the TTC benchmark, three extent sets per permutation
  struct Group {
    std::vector<int> perm;
    std::vector<int> dims[3];
  };
  const Group groups[] = {
      {{1, 0}, {{7248, 7248}, {43408, 1216}, {1216, 43408}}},
      {{0, 2, 1}, {{368, 384, 384}, {2144, 64, 384}, {368, 64, 2307}}},
      {{1, 0, 2}, {{384, 384, 355}, {2320, 384, 59}, {384, 2320, 59}}},
      {{2, 1, 0}, {{384, 355, 384}, {2320, 59, 384}, {384, 59, 2320}}},
      {{0, 3, 2, 1}, {{80, 96, 75, 96}, {464, 16, 75, 96}, {80, 16, 75, 582}}},
      {{2, 1, 3, 0}, {{96, 75, 96, 75}, {608, 12, 96, 75}, {96, 12, 608, 75}}},
      {{2, 0, 3, 1}, {{96, 75, 96, 75}, {608, 12, 96, 75}, {96, 12, 608, 75}}},
      {{1, 0, 3, 2}, {{96, 96, 75, 75}, {608, 96, 12, 75}, {96, 608, 12, 75}}},
      {{3, 2, 1, 0}, {{96, 75, 75, 96}, {608, 12, 75, 96}, {96, 12, 75, 608}}},
      {{0, 4, 2, 1, 3}, {{32, 48, 28, 28, 48}, {176, 8, 28, 28, 48}, {32, 8, 28, 28, 298}}},
      {{3, 2, 1, 4, 0}, {{48, 28, 28, 48, 28}, {352, 4, 28, 48, 28}, {48, 4, 28, 352, 28}}},
      {{2, 0, 4, 1, 3}, {{48, 28, 48, 28, 28}, {352, 4, 48, 28, 28}, {48, 4, 352, 28, 28}}},
      {{1, 3, 0, 4, 2}, {{48, 48, 28, 28, 28}, {352, 48, 4, 28, 28}, {48, 352, 4, 28, 28}}},
      {{4, 3, 2, 1, 0}, {{48, 28, 28, 28, 48}, {352, 4, 28, 28, 48}, {48, 4, 28, 28, 352}}},
      {{0, 3, 2, 5, 4, 1}, {{16, 32, 15, 32, 15, 15}, {48, 10, 15, 32, 15, 15}, {16, 10, 15, 103, 15, 15}}},
      {{3, 2, 0, 5, 1, 4}, {{32, 15, 15, 32, 15, 15}, {112, 5, 15, 32, 15, 15}, {32, 5, 15, 112, 15, 15}}},
      {{2, 0, 4, 1, 5, 3}, {{32, 15, 32, 15, 15, 15}, {112, 5, 32, 15, 15, 15}, {32, 5, 112, 15, 15, 15}}},
      {{3, 2, 5, 1, 0, 4}, {{32, 15, 15, 32, 15, 15}, {112, 5, 15, 32, 15, 15}, {32, 5, 15, 112, 15, 15}}},
      {{5, 4, 3, 2, 1, 0}, {{32, 15, 15, 15, 15, 32}, {112, 5, 15, 15, 15, 32}, {32, 5, 15, 15, 15, 112}}},
  };
  for (const Group& g : groups)
    for (const std::vector<int>& dim : g.dims) {
      if (!benchTensor(dim, g.perm)) return false;
      long long vol = volumeOf(dim);
      std::printf("bandwidth %4.2f GiB/s\n", 2.0 * (double)vol * (double)elemSize / (stats->lastMs() * 1e-3) / 1073741824.0);
    }
  return true;
}

bool bench7(Rng& rng) {
  int samples = samplesOverride ? samplesOverride : 500;
  const std::vector<int> shapes[] = {{5, 3, 2, 4, 35, 33, 37, 40}, {2, 3, 4, 3, 2, 2, 3, 2, 20, 18, 22, 24}};
  for (std::vector<int> dim : shapes) {
    if (volumeOf(dim) > dataElems) {
      std::printf("bench7: shape of %lld elements skipped, buffers hold %lld\n", volumeOf(dim), dataElems);
      continue;
    }
    int rank = (int)dim.size();
    std::vector<int> perm(rank);
    for (int r = 0; r < rank; r++) perm[r] = rank - 1 - r;
    if (!benchTensor(dim, perm)) return false;
    for (int r = 0; r < rank; r++) perm[r] = r;
    for (int s = 0; s < samples; s++) {
      rng.shuffle(dim);
      rng.shuffle(perm);
      if (!isIdentity(perm) && !benchTensor(dim, perm)) return false;
    }
  }
  return true;
}

bool benchMemcpy(long long numElem) {
  if (numElem < 1 || numElem > dataElems) {
    std::printf("memcpy benchmark: element count must be within 1..%lld\n", dataElems);
    return false;
  }
  size_t bytes = (size_t)numElem * elemSize;
  int dim[1] = {(int)numElem}, perm[1] = {0};
  struct Variant {
    const char* name;
    int id;
  };
  const Variant variants[] = {{"copyPerLane", 0}, {"copyVector16", 1}, {"copySmallBlocks", 2}, {"hipMemcpyDtoD", 3}};
  for (const Variant& v : variants) {
    BwStats t(elemSize);
    double sum = 0, best = 0;
    for (int i = 0; i < 4; i++) {
      checker->fillBytes(dataOut, 0xff, bytes);
      HIP_CHECK(hipDeviceSynchronize());
      t.start(0);
      switch (v.id) {
        case 0: copyPerLane(dataIn, dataOut, bytes, elemSize, nullptr); break;
        case 1: copyVector16(dataIn, dataOut, bytes, nullptr); break;
        case 2: copySmallBlocks(dataIn, dataOut, bytes, nullptr); break;
        default: HIP_CHECK(hipMemcpyAsync(dataOut, dataIn, bytes, hipMemcpyDeviceToDevice, 0)); break;
      }
      t.stop(0);
      std::printf("%4.2f GB/s\n", t.gbs(numElem));
      sum += t.gbs(numElem);
      best = std::max(best, t.gbs(numElem));
    }
    if (numElem <= 2147483647LL && !checker->checkAndReport(1, dim, perm, elemSize, dataOut)) return false;
    std::printf("%s average %f GB/s best %f GB/s\n", v.name, sum / 4, best);
  }
  return true;
}

void printDeviceInfo() {
  int dev = 0;
  HIP_CHECK(hipGetDevice(&dev));
  hipDeviceProp_t p;
  HIP_CHECK(hipGetDeviceProperties(&p, dev));
  std::printf("Using %s (%s)\n", p.name, p.gcnArchName);
  std::printf("Clock %1.3f GHz, %d CUs, wavefront %d, LDS per workgroup %zu KB, L2 %1.2f MB, memory %1.1f GB\n",
              (double)p.clockRate / 1e6, p.multiProcessorCount, p.warpSize, p.sharedMemPerBlock / 1024,
              (double)p.l2CacheSize / (1024.0 * 1024.0), (double)p.totalGlobalMem / 1e9);
}

void usage() {
  std::printf("cutt_bench [options]\n");
  std::printf("Options:\n");
  std::printf("-device [int]    : GPU ID (default is 0)\n");
  std::printf("-measure         : use cuttPlanMeasure (default is cuttPlan)\n");
  std::printf("-plantimer       : planning is timed (default is no)\n");
  std::printf("-seed [int]      : seed value for random number generator (default is 1)\n");
  std::printf("-elemsize [int]  : size of elements in bytes, 4 or 8. (default is 8)\n");
  std::printf("-dim ...         : space-separated list of dimensions\n");
  std::printf("-permutation ... : space-separated list of permutations\n");
  std::printf("-bench benchID   : benchmark to run: 3, 5RR (RR = extent ratio, e.g. 510), 6 or 7\n");
  std::printf("-memcpy [int]    : time plain copies of this many elements\n");
  std::printf("-samples [int]   : tensors per rank (bench 3, 5) or per shape (bench 7) instead of the full count\n");
  std::printf("-nomemcpy        : do not time a same-size hipMemcpy beside each tensor\n");
  std::printf("-bufelems [int]  : elements per buffer (default 420M of 4 bytes or 370M of 8 bytes)\n");
  std::printf("-elems [int]     : (average) tensor volume of bench 3 and 5 (default 200M elements)\n");
}

}  // namespace

int main(int argc, char* argv[]) {
  int gpuid = -1, benchID = 0;
  uint64_t seed = 1;
  long long memcpyElems = 0, bufElemsArg = 0, avgElems = 200 * kMillion;
  std::vector<int> dimArg, permArg;
  bool argOk = true;
  int i = 1;
  while (i < argc && argOk) {
    std::string a = argv[i];
    auto intList = [&](std::vector<int>& v) {
      i++;
      while (i < argc && std::isdigit((unsigned char)argv[i][0])) v.push_back(std::atoi(argv[i++]));
    };
    if (a == "-device" && i + 1 < argc) {
      gpuid = std::atoi(argv[i + 1]);
      i += 2;
    } else if (a == "-bench" && i + 1 < argc) {
      benchID = std::atoi(argv[i + 1]);
      i += 2;
    } else if (a == "-measure") {
      useMeasure = true;
      i++;
    } else if (a == "-plantimer") {
      usePlanTimer = true;
      i++;
    } else if (a == "-nomemcpy") {
      timeMemcpy = false;
      i++;
    } else if (a == "-seed" && i + 1 < argc) {
      seed = std::strtoull(argv[i + 1], nullptr, 10);
      i += 2;
    } else if (a == "-samples" && i + 1 < argc) {
      samplesOverride = std::atoi(argv[i + 1]);
      i += 2;
    } else if (a == "-memcpy" && i + 1 < argc) {
      memcpyElems = std::atoll(argv[i + 1]);
      i += 2;
    } else if (a == "-elems" && i + 1 < argc) {
      avgElems = std::atoll(argv[i + 1]);
      i += 2;
    } else if (a == "-bufelems" && i + 1 < argc) {
      bufElemsArg = std::atoll(argv[i + 1]);
      i += 2;
    } else if (a == "-elemsize" && i + 1 < argc) {
      elemSize = (size_t)std::atoi(argv[i + 1]);
      i += 2;
    } else if (a == "-dim") {
      intList(dimArg);
    } else if (a == "-permutation") {
      intList(permArg);
    } else {
      argOk = false;
    }
  }
  if (elemSize != 4 && elemSize != 8) argOk = false;
  if (avgElems < 64) argOk = false;
  if (dimArg.size() != permArg.size()) argOk = false;
  bool known = benchID == 3 || benchID / 100 == 5 || benchID == 6 || benchID == 7;
  if (dimArg.empty() && !known && memcpyElems <= 0) argOk = false;
  if (!argOk) {
    usage();
    return 1;
  }
  if (gpuid >= 0) HIP_CHECK(hipSetDevice(gpuid));
  printDeviceInfo();

  // the reference's buffer sizes: 420M 4-byte or 370M 8-byte elements
  dataElems = (elemSize == 4 ? 420 : 370) * kMillion;
  if (bufElemsArg > 0) dataElems = bufElemsArg;
  HIP_CHECK(hipMalloc(&dataIn, (size_t)dataElems * elemSize));
  HIP_CHECK(hipMalloc(&dataOut, (size_t)dataElems * elemSize));
  checker = new TensorChecker();
  checker->fillPattern(dataIn, (size_t)dataElems * elemSize / 4);
  stats = new BwStats(elemSize);
  copyStats = new BwStats(elemSize);
  Rng rng(seed);

  // The first launch of a process loads the library's code object; keep that out of the timings.
  {
    int wdim[3] = {64, 8, 64}, wperm[3] = {2, 1, 0};
    for (int method : {CUTT_METHOD_TILED, CUTT_METHOD_PACKED}) {
      const int before = cuttGetMethodOverride();
      cuttSetMethodOverride(method);
      cuttHandle warm;
      if (cuttPlan(&warm, 3, wdim, wperm, elemSize, 0) == CUTT_SUCCESS) {
        CUTT_CHECK(cuttExecute(warm, dataIn, dataOut));
        HIP_CHECK(hipDeviceSynchronize());
        CUTT_CHECK(cuttDestroy(warm));
      }
      cuttSetMethodOverride(before);
    }
  }

  bool ok;
  bool withData = true;
  if (!dimArg.empty()) {
    ok = benchTensor(dimArg, permArg);
    if (ok) {
      std::vector<double> v = stats->all();
      std::printf("bandwidth %4.2f GB/s (best of %zu)\n", *std::max_element(v.begin(), v.end()), v.size());
    }
    withData = false;
  } else if (benchID == 3) {
    ok = bench3(rng, avgElems);
    withData = false;
  } else if (benchID / 100 == 5) {
    ok = bench5(rng, avgElems, benchID % 100);
  } else if (benchID == 6) {
    ok = bench6();
  } else if (benchID == 7) {
    ok = bench7(rng);
  } else {
    ok = benchMemcpy(memcpyElems);
  }

  if (ok && !stats->empty() && dimArg.empty()) {
    std::printf("bench%d:\n", benchID);
    stats->printSummary(withData);
  }
  if (ok && !pctOfMemcpy.empty()) {
    std::vector<double> v = pctOfMemcpy;
    std::sort(v.begin(), v.end());
    double sum = 0;
    for (double x : v) sum += x;
    std::printf("percent of same-size hipMemcpy (best of 4 runs each): tensors %zu min %.1f median %.1f mean %.1f max %.1f\n",
                v.size(), v.front(), v[v.size() / 2], sum / v.size(), v.back());
  }
  std::printf(ok ? "bench OK\n" : "bench FAIL\n");
  std::printf("seed %llu\n", (unsigned long long)seed);

  delete stats;
  delete copyStats;
  delete checker;
  HIP_CHECK(hipFree(dataIn));
  HIP_CHECK(hipFree(dataOut));
  return ok ? 0 : 1;
}
