/*
 * cutt_api.cpp - the exported plan API (cutt.h) and its test hooks
 * (cutt_ext.h): input validation, handle table, heuristic and measured plan
 * selection.  Pure host C++; the GPU is reached through hip_layer.h.
 *
 * Mirrors the behaviour of reference src/cutt.cpp:36-310.  Deliberate
 * differences: the handle table is guarded by a mutex (the reference's
 * globals are unguarded, src/cutt.cpp:36-42); a HIP failure becomes
 * CUTT_INTERNAL_ERROR instead of exit(1) (reference src/CudaUtils.h:35-42);
 * cuttPlanMeasure times each candidate twice and keeps the faster run,
 * because a first launch also pays for loading the kernel.
 */
#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <list>
#include <memory>
#include <mutex>
#include <string>
#include <system_error>
#include <thread>
#include <unordered_map>
#include <vector>

#include "../../include/cutt_ext.h"
#include "hip_layer.h"
#include "model.h"
#include "plan.h"
#include "slab.h"

using namespace cutt;

namespace {

struct StoredPlan {
  Plan plan;
  // A tensor beyond what one launch addresses (slab.h): one launch per piece, with the plan of the
  // piece's shape - `plan` for shape 0, more[s - 1] for shape s.  Empty for every other tensor.
  std::vector<Plan> more;
  std::vector<SlabPiece> pieces;
  int numCandidates = 0;
  double planMs = 0;
  double usMeasured = 0;
};

std::mutex gMutex;
// A handle maps to a shared owner: cuttExecute copies the pointer under the mutex and launches from
// its copy, so a cuttDestroy of the same handle from another thread frees the plan (and its device
// tables) only after that launch has been issued.
std::unordered_map<cuttHandle, std::shared_ptr<StoredPlan>> gPlans;
cuttHandle gNextHandle = 0;
std::unordered_map<int, cuttHipDeviceProps> gDeviceProps;
int gMethodOverride = -1;  // -1 = not initialised from the environment yet
std::vector<cuttPlanInfo> gLastMeasurement;

// What cuttPlan decided for the problems it saw last, most recent first: a second cuttPlan for the
// same tensor on the same device copies the decision instead of enumerating and estimating the
// candidates again.  Entries hold host data only (no device tables, no stream).
struct CachedDecision {
  std::string key;
  Plan plan;
  int numCandidates;
};
std::list<CachedDecision> gDecisions;
std::unordered_map<std::string, std::list<CachedDecision>::iterator> gDecisionIndex;

// Entries the cache may hold: CUTT_PLAN_CACHE (default 64; 0 switches it off).
size_t planCacheCapacity() {
  if (const char* e = std::getenv("CUTT_PLAN_CACHE")) return (size_t)std::max(0, std::atoi(e));
  return 64;
}

// Everything a decision depends on: device, method override, the tensor, and the tuning variables
// of the environment as they are now.
std::string planKey(int deviceID, int force, int rank, const int* dim, const int* perm, size_t sizeofType) {
  std::string k;
  auto put = [&](long long v) {
    k += std::to_string(v);
    k += ',';
  };
  put(deviceID); put(force); put((long long)sizeofType); put(rank);
  for (int i = 0; i < rank; i++) put(dim[i]);
  for (int i = 0; i < rank; i++) put(perm[i]);
  for (const char* name : {"CUTT_TILED_ORDER", "CUTT_XCD_AWARE", "CUTT_ELEMS_PER_THREAD", "CUTT_PACKED_ROUNDS",
                           "CUTT_MAX_ITEMS", "CUTT_ITEM_ORDER", "CUTT_PAD_SHIFT", "CUTT_CACHE_POLICY", "CUTT_WIDE_OFFSETS", "CUTT_MBAR_ORDER",
                           "CUTT_SUPER_M", "CUTT_SUPER_K", "CUTT_TILED_GROUPED", "CUTT_TILED_ALIGNED", "CUTT_TILE_DIGITS", "CUTT_ITEM_DIGITS", "CUTT_DIGIT_LANES", "CUTT_TILED_FUSE", "CUTT_ADDRESS_BITS", "CUTT_MODEL_RUN_LENGTH"}) {
    const char* e = std::getenv(name);
    k += e ? e : "-";
    k += ';';
  }
  return k;
}

bool planCacheLookup(const std::string& key, Plan& out, int& numCandidates) {
  std::lock_guard<std::mutex> lock(gMutex);
  auto it = gDecisionIndex.find(key);
  if (it == gDecisionIndex.end()) return false;
  gDecisions.splice(gDecisions.begin(), gDecisions, it->second);  // most recent first
  out = it->second->plan.clone();
  numCandidates = it->second->numCandidates;
  return true;
}

void planCacheInsert(const std::string& key, const Plan& chosen, int numCandidates) {
  const size_t capacity = planCacheCapacity();
  std::lock_guard<std::mutex> lock(gMutex);
  if (capacity == 0 || gDecisionIndex.count(key)) return;
  gDecisions.push_front(CachedDecision{key, chosen.clone(), numCandidates});
  gDecisionIndex[key] = gDecisions.begin();
  while (gDecisions.size() > capacity) {
    gDecisionIndex.erase(gDecisions.back().key);
    gDecisions.pop_back();
  }
}

int methodOverrideLocked() {
  if (gMethodOverride < 0) {
    gMethodOverride = 0;
    const char* e = std::getenv("CUTT_FORCE_METHOD");
    if (e) {
      std::string s(e);
      for (char& c : s) c = (char)std::tolower((unsigned char)c);
      if (s == "tiled") gMethodOverride = kTiled;
      else if (s == "tiledcopy") gMethodOverride = kTiledCopy;
      else if (s == "packed") gMethodOverride = kPacked;
      else if (s == "packedsplit") gMethodOverride = kPackedSplit;
    }
  }
  return gMethodOverride;
}

// Largest rank the API accepts.  One launch handles at most CUTT_MAX_RANK ranks and 2^32 - 1
// elements (element offsets are unsigned 32-bit in the kernels, byte addresses 64-bit); a tensor
// beyond either is cut into pieces within those limits (slab.h).
constexpr int kMaxApiRank = 64;
constexpr long long kMaxElements = 1ll << 46;

// Same checks as reference src/cutt.cpp:59-82 (whose int arithmetic implies fewer than 2^31
// elements).  `large` receives whether the tensor has to be cut into pieces; an entry point that
// passes none refuses such tensors.
cuttResult checkInput(int rank, const int* dim, const int* perm, size_t sizeofType, bool* large = nullptr) {
  if (sizeofType != 4 && sizeofType != 8) return CUTT_INVALID_PARAMETER;
  if (rank <= 1 || rank > kMaxApiRank) return CUTT_INVALID_PARAMETER;
  if (!dim || !perm) return CUTT_INVALID_PARAMETER;
  long long vol = 1;
  for (int i = 0; i < rank; i++) {
    if (dim[i] <= 1) return CUTT_INVALID_PARAMETER;
    vol *= dim[i];
    if (vol > kMaxElements) return CUTT_INVALID_PARAMETER;
  }
  const bool cut = rank > CUTT_MAX_RANK || slabNeeded(rank, dim, slabSpanLimit());
  if (cut && !large) return CUTT_INVALID_PARAMETER;
  if (large) *large = cut;
  std::vector<char> seen(rank, 0);
  for (int i = 0; i < rank; i++) {
    if (perm[i] < 0 || perm[i] >= rank || seen[perm[i]]) return CUTT_INVALID_PARAMETER;
    seen[perm[i]] = 1;
  }
  return CUTT_SUCCESS;
}

bool currentDevice(int& deviceID, cuttHipDeviceProps& props) {
  if (cuttHipGetDevice(&deviceID) != 0) return false;
  std::lock_guard<std::mutex> lock(gMutex);
  auto it = gDeviceProps.find(deviceID);
  if (it == gDeviceProps.end()) {
    cuttHipDeviceProps p;
    if (cuttHipGetDeviceProps(deviceID, &p) != 0) return false;
    sanitizeDeviceProps(p);
    it = gDeviceProps.emplace(deviceID, p).first;
  }
  props = it->second;
  return true;
}

void fillInfo(const Plan& p, cuttPlanInfo& o) {
  std::memset(&o, 0, sizeof(o));
  o.method = p.method;
  o.fromReduced = p.fromReduced;
  o.rank = p.pb.rank;
  o.numMm = p.split.numMm;
  o.numMk = p.split.numMk;
  o.splitRank = p.split.splitRank[0];
  o.splitDim = p.split.splitDim[0];
  o.numSplit = p.split.numSplit[0];
  o.splitRank2 = p.split.splitRank[1];
  o.splitDim2 = p.split.splitDim[1];
  o.numSplit2 = p.split.numSplit[1];
  o.volMm = p.split.volMm;
  o.volMk = p.split.volMk;
  o.volMmk = p.split.volMmk;
  o.volMbar = p.split.volMbar;
  o.volMmkInCont = p.split.volMmkInCont;
  o.volMmkOutCont = p.split.volMmkOutCont;
  o.volMmkUnsplit = p.split.volMmkUnsplit;
  o.numBlocks = p.numBlocks;
  o.numThreads = p.numThreads;
  o.itemsPerBlock = p.packed.itemsPerBlock;
  o.tiledOrder = p.method == kTiled ? p.tiled.order : p.tcopy.order;
  o.ldsBytes = p.ldsBytes;
  o.usPredicted = p.model.usPredicted;
  o.rdLines = p.model.rdLines;
  o.wrLines = p.model.wrLines;
  o.rdInstr = p.model.rdInstr;
  o.wrInstr = p.model.wrInstr;
  o.wrPartialLines = p.model.wrPartialLines;
  o.rdSectors = p.model.rdSectors;
  o.wrSectors = p.model.wrSectors;
  o.ldsCycles = p.model.ldsCycles;
  o.blocksPerCU = p.model.blocksPerCU;
  o.cachePolicy = p.method == kTiled ? p.tiled.cachePolicy
                                      : (p.method == kTiledCopy ? p.tcopy.cachePolicy : p.packed.cachePolicy);
  o.elemsPerThread = p.packed.elemsPerThread;
  o.tiledGrouped = p.method == kTiled ? p.tiled.grouped : 0;
  o.tiledAligned = p.method == kTiled ? p.tiled.alignedStores : 0;
  o.itemOrder = (p.method == kPacked || p.method == kPackedSplit) ? p.packed.itemOrder : 0;
  o.numPieces = 1;
  o.numShapes = 1;
  o.wideOffsets = (p.method == kPacked || p.method == kPackedSplit) ? p.packed.wideOffsets : 0;
  o.superM = p.method == kTiled ? (int)p.tiled.superM : (p.method == kTiledCopy ? (int)p.tcopy.superM : 0);
  o.superK = p.method == kTiled ? (int)p.tiled.superK : (p.method == kTiledCopy ? (int)p.tcopy.superK : 0);
  o.rdEdgeDist = p.model.rdEdgeDist;
  o.wrEdgeDist = p.model.wrEdgeDist;
  std::memset(o.tileDigits, 0, sizeof(o.tileDigits));
  if ((p.method == kTiled || p.method == kTiledCopy) && o.tiledOrder == 7) {
    const std::string t = formatTileDigits(p.method == kTiled ? p.tiled.digits : p.tcopy.digits);
    std::strncpy(o.tileDigits, t.c_str(), sizeof(o.tileDigits) - 1);
  } else if ((p.method == kPacked || p.method == kPackedSplit) && p.itemDigits.n > 0) {
    const std::string t = formatTileDigits(p.itemDigits);
    std::strncpy(o.tileDigits, t.c_str(), sizeof(o.tileDigits) - 1);
  }
}

void setCachePolicy(Plan& p, int policy) {
  p.tiled.cachePolicy = policy;
  p.tcopy.cachePolicy = policy;
  p.packed.cachePolicy = policy;
}

int cachePolicyOf(const Plan& p) {
  if (p.method == kTiled) return p.tiled.cachePolicy;
  if (p.method == kTiledCopy) return p.tcopy.cachePolicy;
  return p.packed.cachePolicy;
}

// Cache policy from the model's sampled address stream.  Streaming loads give up the L2 copy of a
// line, so they pay off only when a workgroup uses (nearly) whole lines of what it reads;
// streaming stores only when no written line is left partly covered by a workgroup.
// (Not applied when CUTT_CACHE_POLICY pins the policy.)
void chooseCachePolicy(Plan& p, const cuttHipDeviceProps& props) {
  if (std::getenv("CUTT_CACHE_POLICY")) return;
  // The memory-side cache decides for small and medium tensors (measured on random tensors of
  // 4M-200M elements): while input and output fit it together, ordinary accesses are best
  // (non-temporal ones go past it: 65-72 % of memcpy instead of 80-89 %); up to about 3.5 times
  // its size per buffer, streaming the reads and letting the cache merge the writes wins clearly
  // (at one cache size per buffer 99 % against 81 %); beyond that it no longer matters.
  const double bytes = (double)p.pb.volume * p.pb.elemSize;
  const double cache = (double)props.infinityCacheBytes;
  if (cache > 0 && 2.0 * bytes <= cache) {
    setCachePolicy(p, 0);
    return;
  }
  const double lines = bytes / 128.0;
  if (cache > 0 && bytes <= 3.5 * cache) {
    // ... unless the plan reads each line from several requests (more than ~1.7 lines requested
    // per line of data): then the re-reads must find the line in the caches (0.85-0.97 x).
    // A Tiled plan's 256-byte rows of 4-byte elements share every third line with the neighbouring
    // tile: there the limit is 1.5, except between 0.8 and 1.8 cache sizes per buffer, where it is
    // 1.6 (at 1.56 lines per line of data: ordinary loads +10 % at 0.75 cache sizes and +7...+15 %
    // at 2.1-3.1, streaming loads +9...+18 % at 0.88-1.56), and a plan that keeps four rows per
    // lane in flight always streams its reads (+2...+24 % over ordinary loads at 1-3.4 cache sizes).
    const bool narrowTiles = (p.method == kTiled || p.method == kTiledCopy) && p.pb.elemSize == 4;
    const double limit = narrowTiles ? (bytes >= 0.8 * cache && bytes < 1.8 * cache ? 1.6 : 1.5) : 1.7;
    const bool grouped = p.method == kTiled && p.tiled.grouped;
    setCachePolicy(p, grouped || p.model.rdLines < limit * lines ? 1 : 0);
    return;
  }
  const bool wholeReads = p.model.rdLines <= 1.15 * lines;
  const bool wholeWrites = p.model.wrPartialLines == 0.0;
  setCachePolicy(p, wholeReads ? (wholeWrites ? 3 : 1) : 0);
}

// Runs f(0) .. f(n-1) on up to eight host threads (CUTT_PLAN_THREADS caps the number; 1 = the
// calling thread only) and returns when all have finished; false if a call threw (out of memory).
// The calls must not depend on each other: the model's estimate of a candidate is a pure function
// of that candidate, so a plan does not depend on the number of threads.
template <class F>
bool parallelFor(int n, F&& f) {
  int cap = 8;
  if (const char* e = std::getenv("CUTT_PLAN_THREADS")) cap = std::max(1, std::atoi(e));
  const unsigned hw = std::thread::hardware_concurrency();
  const int nt = std::min({n, cap, hw ? (int)hw : 1});
  std::atomic<int> next{0};
  std::atomic<bool> threw{false};
  auto work = [&]() {
    for (int i = next.fetch_add(1); i < n; i = next.fetch_add(1)) {
      try {
        f(i);
      } catch (...) {
        threw = true;
      }
    }
  };
  std::vector<std::thread> helpers;
  for (int t = 1; t < nt; t++) {
    try {
      helpers.emplace_back(work);
    } catch (const std::system_error&) {
      break;  // no more threads to be had: the calling thread does the rest
    }
  }
  work();
  for (std::thread& t : helpers) t.join();
  return !threw;
}

// A Tiled plan on 4-byte elements whose tile rows start off the 128-byte grid (the model counts
// 1.2-1.6 requested lines per line of data on both sides) and whose tensor is larger than the
// memory-side cache (from 1.1 cache sizes per buffer on) keeps four instead of sixteen rows per
// lane in flight.  Measured on such plans of the reference's random-tensor suites: +5 % in the
// median at 0.8 GB per buffer (164 plans, worst -3.5 %, best +17 %), single tensors +20...+34 % at
// 0.3-0.5 GB; outside these limits the same switch costs up to 14 % (aligned or cache-sized
// tensors, 8-byte elements).  (Not applied when CUTT_TILED_GROUPED pins the switch.)
void chooseTiledGrouping(Plan& p, const cuttHipDeviceProps& props) {
  if (p.method != kTiled || std::getenv("CUTT_TILED_GROUPED") || p.tiled.alignedStores) return;
  const double bytes = (double)p.pb.volume * p.pb.elemSize;
  const double lines = bytes / 128.0;
  const double cache = props.infinityCacheBytes > 0 ? (double)props.infinityCacheBytes : 256.0 * 1024 * 1024;
  const double rdAmp = p.model.rdLines / lines, wrAmp = p.model.wrLines / lines;
  const bool grouped = p.pb.elemSize == 4 && bytes > 1.1 * cache && rdAmp > 1.2 && rdAmp < 1.6 && wrAmp > 1.2 &&
                       wrAmp < 1.6;
  p.tiled.grouped = grouped ? 1 : 0;
  if (grouped) p.model.usPredicted *= 0.96;
}

// The model's estimate of a candidate and the launch details that follow from it.
bool estimateAndTune(Plan& p, const cuttHipDeviceProps& props) {
  if (!estimatePlan(p, props, 10)) return false;
  chooseTiledGrouping(p, props);
  return true;
}

// Model estimate of every candidate; false if one of them fails.
bool estimateAll(std::vector<Plan>& plans, const cuttHipDeviceProps& props) {
  std::atomic<bool> ok{true};
  const bool ran = parallelFor((int)plans.size(), [&](int i) {
    if (!estimateAndTune(plans[i], props)) ok = false;
  });
  return ran && ok;
}

PlannerOptions plannerOptions(int forceMethod);

// The order in which consecutive work items walk the Mbar ranks decides whether the lines shared
// by neighbouring runs meet in the L2 on the read side or on the write side.  For the few
// candidates the model ranks best, also estimate the other orders and keep the cheapest.
// (Not applied when CUTT_MBAR_ORDER pins the order.)
void refineMbarOrder(std::vector<Plan>& plans, const cuttHipDeviceProps& props, int force) {
  if (std::getenv("CUTT_MBAR_ORDER")) return;
  const PlannerOptions base = plannerOptions(force);
  std::vector<int> idx;
  for (int i = 0; i < (int)plans.size(); i++)
    if (plans[i].method != kTrivial) idx.push_back(i);
  std::sort(idx.begin(), idx.end(),
            [&](int a, int b) { return plans[a].model.usPredicted < plans[b].model.usPredicted; });
  struct Trial {
    int plan, order;
    bool ok;
    Plan q;
  };
  std::vector<Trial> trials;
  for (size_t k = 0; k < idx.size() && k < 3; k++)
    for (int order : {0, 1, 2})
      if (order != base.mbarOrder) trials.push_back({idx[k], order, false, Plan()});
  // a trial that fails or throws keeps ok == false and is passed over
  (void)parallelFor((int)trials.size(), [&](int i) {
    Trial& t = trials[i];
    PlannerOptions opt = base;
    opt.mbarOrder = t.order;
    t.ok = rebuildPlan(plans[t.plan], props, opt, t.q) && estimateAndTune(t.q, props);
  });
  for (Trial& t : trials) {
    Plan& p = plans[t.plan];
    if (t.ok && t.q.model.usPredicted < p.model.usPredicted) p = std::move(t.q);
  }
}

// Index of the candidate with the smallest predicted time; Trivial always wins and ties go to
// the later candidate (reference src/cuttplan.cpp:700-768).
int chooseHeuristic(const std::vector<Plan>& plans) {
  int best = -1;
  for (int i = 0; i < (int)plans.size(); i++) {
    if (plans[i].method == kTrivial) return i;
    if (best < 0 || plans[i].model.usPredicted <= plans[best].model.usPredicted) best = i;
  }
  return best;
}

PlannerOptions plannerOptions(int forceMethod) {
  PlannerOptions opt;
  opt.forceMethod = forceMethod;
  // Tuning knobs for experiments; the defaults are what the library ships with.
  if (const char* e = std::getenv("CUTT_TILED_ORDER")) opt.tiledOrder = std::atoi(e);
  if (const char* e = std::getenv("CUTT_XCD_AWARE")) opt.xcdAware = std::atoi(e) != 0;
  if (const char* e = std::getenv("CUTT_ELEMS_PER_THREAD")) {
    const int v = std::atoi(e);
    if (v == 1 || v == 2 || v == 4 || v == 8 || v == 16) opt.elemsPerThread = v;
  }
  if (const char* e = std::getenv("CUTT_PACKED_ROUNDS")) opt.packedRounds = std::max(0, std::atoi(e));
  if (const char* e = std::getenv("CUTT_PAD_SHIFT")) opt.padShift = std::min(31, std::max(1, std::atoi(e)));
  if (const char* e = std::getenv("CUTT_ITEM_ORDER")) opt.itemOrder = std::min(2, std::max(0, std::atoi(e)));
  if (const char* e = std::getenv("CUTT_MAX_ITEMS")) opt.maxItemsPerBlock = std::max(1, std::atoi(e));
  if (const char* e = std::getenv("CUTT_CACHE_POLICY")) {
    const int v = std::atoi(e);
    if (v == 0 || v == 1 || v == 3) opt.cachePolicy = v;
  }
  if (const char* e = std::getenv("CUTT_WIDE_OFFSETS")) opt.wideOffsets = std::atoi(e) != 0;
  if (const char* e = std::getenv("CUTT_MBAR_ORDER")) opt.mbarOrder = std::atoi(e);
  if (const char* e = std::getenv("CUTT_SUPER_M")) { opt.superM = std::max(1, std::atoi(e)); opt.superAuto = false; }
  if (const char* e = std::getenv("CUTT_SUPER_K")) { opt.superK = std::max(1, std::atoi(e)); opt.superAuto = false; }
  if (const char* e = std::getenv("CUTT_TILED_GROUPED")) opt.tiledGrouped = std::atoi(e) != 0 ? 1 : 0;
  if (const char* e = std::getenv("CUTT_TILED_ALIGNED")) opt.tiledAligned = std::atoi(e) != 0 ? 1 : 0;
  if (const char* e = std::getenv("CUTT_TILE_DIGITS")) opt.tileDigits = e;
  if (const char* e = std::getenv("CUTT_ITEM_DIGITS")) opt.itemDigits = e;
  if (const char* e = std::getenv("CUTT_DIGIT_LANES")) opt.digitLanes = std::atoi(e) != 0 ? 1 : 0;
  if (const char* e = std::getenv("CUTT_TILED_FUSE")) opt.tiledFuse = std::atoi(e) != 0 ? 1 : 0;
  if (const char* e = std::getenv("CUTT_ADDRESS_BITS")) opt.addressBits = std::atoi(e) != 0;
  return opt;
}

// The problem as given and with its ranks fused.
void makeProblems(int rank, const int* dim, const int* perm, size_t sizeofType, Problem& orig, Problem& red) {
  orig.set(rank, dim, perm, (int)sizeofType);
  std::vector<int> redDim, redPerm;
  reduceRanks(rank, dim, perm, redDim, redPerm);
  red.set((int)redDim.size(), redDim.data(), redPerm.data(), (int)sizeofType);
}

bool enumerate(int rank, const int* dim, const int* perm, size_t sizeofType,
               const cuttHipDeviceProps& props, int forceMethod, std::vector<Plan>& plans) {
  Problem orig, red;
  makeProblems(rank, dim, perm, sizeofType, orig, red);
  return createPlans(orig, red, props, plannerOptions(forceMethod), plans);
}

cuttResult storePlan(cuttHandle* handle, Plan&& chosen, void* stream, int deviceID, int numCandidates,
                     double usMeasured, std::chrono::steady_clock::time_point t0) {
  std::shared_ptr<StoredPlan> sp = std::make_shared<StoredPlan>();
  sp->plan = std::move(chosen);
  sp->plan.stream = stream;
  sp->plan.deviceID = deviceID;
  sp->numCandidates = numCandidates;
  sp->usMeasured = usMeasured;
  if (sp->plan.activate() != 0) return CUTT_INTERNAL_ERROR;
  sp->planMs = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  std::lock_guard<std::mutex> lock(gMutex);
  *handle = gNextHandle++;
  if (gPlans.count(*handle)) return CUTT_INTERNAL_ERROR;
  gPlans.emplace(*handle, std::move(sp));
  return CUTT_SUCCESS;
}

// The same for a tensor in pieces: parts[s] is the plan of the pieces of shape s.
cuttResult storeLargePlan(cuttHandle* handle, std::vector<Plan>&& parts, std::vector<SlabPiece>&& pieces, void* stream,
                          int deviceID, int numCandidates, double usMeasured,
                          std::chrono::steady_clock::time_point t0) {
  std::shared_ptr<StoredPlan> sp = std::make_shared<StoredPlan>();
  for (Plan& p : parts) {
    p.stream = stream;
    p.deviceID = deviceID;
    if (p.activate() != 0) return CUTT_INTERNAL_ERROR;
  }
  sp->plan = std::move(parts[0]);
  for (size_t s = 1; s < parts.size(); s++) sp->more.push_back(std::move(parts[s]));
  sp->pieces = std::move(pieces);
  sp->numCandidates = numCandidates;
  sp->usMeasured = usMeasured;
  sp->planMs = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  std::lock_guard<std::mutex> lock(gMutex);
  *handle = gNextHandle++;
  if (gPlans.count(*handle)) return CUTT_INTERNAL_ERROR;
  gPlans.emplace(*handle, std::move(sp));
  return CUTT_SUCCESS;
}

}  // namespace

// What cuttPlan decides for this tensor on this device: from the memory of recent decisions, or by
// enumerating the candidates and ranking them with the cost model.  Host work only.
static cuttResult decideHeuristically(int rank, int* dim, int* permutation, size_t sizeofType, int deviceID,
                                      const cuttHipDeviceProps& props, Plan& chosen, int& numCandidates) {
  int force;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    force = methodOverrideLocked();
  }
  const bool useCache = planCacheCapacity() > 0;
  const std::string key = useCache ? planKey(deviceID, force, rank, dim, permutation, sizeofType) : std::string();
  if (useCache && planCacheLookup(key, chosen, numCandidates)) return CUTT_SUCCESS;
  std::vector<Plan> plans;
  if (!enumerate(rank, dim, permutation, sizeofType, props, force, plans)) return CUTT_INTERNAL_ERROR;
  if (!estimateAll(plans, props)) return CUTT_INTERNAL_ERROR;
  refineMbarOrder(plans, props, force);
  const int best = chooseHeuristic(plans);
  if (best < 0) return CUTT_INTERNAL_ERROR;
  chooseCachePolicy(plans[best], props);
  if (useCache) planCacheInsert(key, plans[best], (int)plans.size());
  numCandidates = (int)plans.size();
  chosen = std::move(plans[best]);
  return CUTT_SUCCESS;
}

struct Measured {
  Plan plan;
  int numCandidates = 0;
  double bestUs = 0;
};
static cuttResult measureProblem(const Problem& orig, const Problem& red, int force, int deviceID,
                                 const cuttHipDeviceProps& props, hipStream_t stream, void* idata, void* odata,
                                 size_t numBytes, Measured& out);

// Elements between the first and the last element of a problem's output, inclusive.
static int64_t outputSpan(const Problem& pb) {
  int64_t span = 1;
  for (int r = 0; r < pb.rank; r++) span += (int64_t)(pb.dim[r] - 1) * pb.strideOut[r];
  return span;
}

// cuttPlan / cuttPlanMeasure for a tensor that one launch cannot address: the fused tensor is cut
// into pieces (slab.h) and every shape of piece is planned like a tensor of its own - by the cost
// model, or by timing its candidates on the first piece of that shape.
static cuttResult planLarge(cuttHandle* handle, int rank, int* dim, int* permutation, size_t sizeofType,
                            hipStream_t stream, bool measure, void* idata, void* odata,
                            std::chrono::steady_clock::time_point t0) {
  int deviceID;
  cuttHipDeviceProps props;
  if (!currentDevice(deviceID, props)) return CUTT_INTERNAL_ERROR;
  int force;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    force = methodOverrideLocked();
  }
  std::vector<int> redDim, redPerm;
  reduceRanks(rank, dim, permutation, redDim, redPerm);
  SlabDecomposition dec;
  if (!slabDecompose((int)redDim.size(), redDim.data(), redPerm.data(), (int)sizeofType, slabSpanLimit(), dec))
    return CUTT_INVALID_PARAMETER;
  std::vector<Plan> parts(dec.shapes.size());
  int numCandidates = 0;
  double usMeasured = 0;
  for (size_t s = 0; s < dec.shapes.size(); s++) {
    const Problem& shape = dec.shapes[s];
    if (shape.rank > CUTT_MAX_RANK) return CUTT_INVALID_PARAMETER;
    if (measure) {
      size_t first = 0;
      while (dec.pieces[first].shape != (int)s) first++;
      Measured m;
      cuttResult r = measureProblem(shape, shape, force, deviceID, props, stream,
                                    (char*)idata + dec.pieces[first].baseIn * (int64_t)sizeofType,
                                    (char*)odata + dec.pieces[first].baseOut * (int64_t)sizeofType,
                                    (size_t)outputSpan(shape) * sizeofType, m);
      if (r != CUTT_SUCCESS) return r;
      parts[s] = std::move(m.plan);
      if (s == 0) { numCandidates = m.numCandidates; usMeasured = m.bestUs; }
    } else {
      std::vector<Plan> plans;
      if (!createPlans(shape, shape, props, plannerOptions(force), plans) || plans.empty()) return CUTT_INTERNAL_ERROR;
      if (!estimateAll(plans, props)) return CUTT_INTERNAL_ERROR;
      refineMbarOrder(plans, props, force);
      const int best = chooseHeuristic(plans);
      if (best < 0) return CUTT_INTERNAL_ERROR;
      chooseCachePolicy(plans[best], props);
      if (s == 0) numCandidates = (int)plans.size();
      parts[s] = std::move(plans[best]);
    }
  }
  return storeLargePlan(handle, std::move(parts), std::move(dec.pieces), (void*)stream, deviceID, numCandidates,
                        usMeasured, t0);
}

static cuttResult planImpl(cuttHandle* handle, int rank, int* dim, int* permutation,
                           size_t sizeofType, hipStream_t stream) {
  const auto t0 = std::chrono::steady_clock::now();
  if (!handle) return CUTT_INVALID_PARAMETER;
  bool large = false;
  cuttResult chk = checkInput(rank, dim, permutation, sizeofType, &large);
  if (chk != CUTT_SUCCESS) return chk;
  if (large) return planLarge(handle, rank, dim, permutation, sizeofType, stream, false, nullptr, nullptr, t0);

  int deviceID;
  cuttHipDeviceProps props;
  if (!currentDevice(deviceID, props)) return CUTT_INTERNAL_ERROR;
  Plan chosen;
  int numCandidates = 0;
  chk = decideHeuristically(rank, dim, permutation, sizeofType, deviceID, props, chosen, numCandidates);
  if (chk != CUTT_SUCCESS) return chk;
  return storePlan(handle, std::move(chosen), (void*)stream, deviceID, numCandidates, 0.0, t0);
}

// cuttPlan + cuttExecute in one call that allocates nothing on the device: the index tables of a
// Packed / PackedSplit plan are built by a kernel on `stream` in the library's static scratch
// memory, then the transpose is launched on the same stream.  See cutt.h.
static cuttResult executeNoAllocImpl(int rank, int* dim, int* permutation, size_t sizeofType, hipStream_t stream,
                                     void* idata, void* odata) {
  cuttResult chk = checkInput(rank, dim, permutation, sizeofType);
  if (chk != CUTT_SUCCESS) return chk;
  if (idata == odata || !idata || !odata) return CUTT_INVALID_PARAMETER;
  int deviceID;
  cuttHipDeviceProps props;
  if (!currentDevice(deviceID, props)) return CUTT_INTERNAL_ERROR;
  Plan plan;
  int numCandidates = 0;
  chk = decideHeuristically(rank, dim, permutation, sizeofType, deviceID, props, plan, numCandidates);
  if (chk != CUTT_SUCCESS) return chk;
  plan.stream = (void*)stream;
  plan.deviceID = deviceID;
  void* scratch = nullptr;
  size_t scratchBytes = 0;
  if (plan.tableBytes() > 0) {
    if (int e = cuttHipScratch(&scratch, &scratchBytes); e != 0) {
      std::fprintf(stderr, "cuttExecuteNoAlloc: no address for the static scratch memory (%s)\n", cuttHipErrorString(e));
      return CUTT_INTERNAL_ERROR;
    }
    if (const char* e = std::getenv("CUTT_NOALLOC_MAX_BYTES"))  // a smaller limit, for tests
      scratchBytes = std::min(scratchBytes, (size_t)std::max(0ll, std::atoll(e)));
    if (plan.tableBytes() > scratchBytes) {
      std::fprintf(stderr, "cuttExecuteNoAlloc: the plan's index tables (%zu bytes) exceed the static scratch "
                           "memory (%zu bytes)\n", plan.tableBytes(), scratchBytes);
      return CUTT_INVALID_PARAMETER;
    }
  }
  if (int e = plan.activateInPlace(scratch, scratchBytes); e != 0) {
    std::fprintf(stderr, "cuttExecuteNoAlloc: building the index tables failed (%d%s%s)\n", e, e > 0 ? " " : "",
                 e > 0 ? cuttHipErrorString(e) : "");
    return CUTT_INTERNAL_ERROR;
  }
  if (int e = plan.launch(idata, odata); e != 0) {
    std::fprintf(stderr, "cuttExecuteNoAlloc: launch failed (%d%s%s)\n", e, e > 0 ? " " : "",
                 e > 0 ? cuttHipErrorString(e) : "");
    return CUTT_INTERNAL_ERROR;
  }
  return CUTT_SUCCESS;
}

static cuttResult planMeasureImpl(cuttHandle* handle, int rank, int* dim, int* permutation,
                                  size_t sizeofType, hipStream_t stream, void* idata, void* odata) {
  const auto t0 = std::chrono::steady_clock::now();
  if (!handle) return CUTT_INVALID_PARAMETER;
  bool large = false;
  cuttResult chk = checkInput(rank, dim, permutation, sizeofType, &large);
  if (chk != CUTT_SUCCESS) return chk;
  if (idata == odata || !idata || !odata) return CUTT_INVALID_PARAMETER;
  if (large) return planLarge(handle, rank, dim, permutation, sizeofType, stream, true, idata, odata, t0);

  int deviceID;
  cuttHipDeviceProps props;
  if (!currentDevice(deviceID, props)) return CUTT_INTERNAL_ERROR;
  int force;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    force = methodOverrideLocked();
  }
  Problem orig, red;
  makeProblems(rank, dim, permutation, sizeofType, orig, red);
  Measured m;
  chk = measureProblem(orig, red, force, deviceID, props, stream, idata, odata, (size_t)orig.volume * sizeofType, m);
  if (chk != CUTT_SUCCESS) return chk;
  return storePlan(handle, std::move(m.plan), (void*)stream, deviceID, m.numCandidates, m.bestUs, t0);
}

// Times the candidates of one problem on the caller's buffers (`numBytes` of the output are
// overwritten before every run) and hands back the fastest, activated.
static cuttResult measureProblem(const Problem& orig, const Problem& red, int force, int deviceID,
                                 const cuttHipDeviceProps& props, hipStream_t stream, void* idata, void* odata,
                                 size_t numBytes, Measured& out) {
  std::vector<Plan> plans;
  if (!createPlans(orig, red, props, plannerOptions(force), plans)) return CUTT_INTERNAL_ERROR;
  if (plans.empty()) return CUTT_INTERNAL_ERROR;
  if (!estimateAll(plans, props)) return CUTT_INTERNAL_ERROR;
  for (Plan& p : plans) chooseCachePolicy(p, props);

  // Candidates the model puts more than twice behind its best are not timed when there are many (the
  // model's worst recorded errors: classes of plans that ran 1.3-1.4 times their estimate, a pick at 0.6 of
  // the measured plan's rate); up to twenty candidates are all timed, as the reference does with any
  // number (src/cutt.cpp:236-262), and CUTT_MEASURE_ALL=1 asks for that always.
  double bestPred = 1e300;
  for (const Plan& p : plans) bestPred = std::min(bestPred, p.model.usPredicted);
  double margin = plans.size() <= 20 ? 1e30 : 2.0;
  if (const char* e = std::getenv("CUTT_MEASURE_ALL"))
    if (std::atoi(e) != 0) margin = 1e30;

  // the two events of the timed runs; destroyed on every way out of this function
  struct Events {
    void *start = nullptr, *stop = nullptr;
    ~Events() {
      if (start) cuttHipEventDestroy(start);
      if (stop) cuttHipEventDestroy(stop);
    }
  } events;
  if (cuttHipEventCreate(&events.start) != 0 || cuttHipEventCreate(&events.stop) != 0) return CUTT_INTERNAL_ERROR;
  void* const evStart = events.start;
  void* const evStop = events.stop;
  double bestUs = 1e300;
  bool failed = false;
  // Times plan p (two runs, the faster counts); returns false on a HIP error.
  auto timePlan = [&](Plan& p, double& t) -> bool {
    p.stream = (void*)stream;
    p.deviceID = deviceID;
    if (p.activate() != 0) return false;
    t = 1e300;
    for (int rep = 0; rep < 2; rep++) {
      // Overwrite the output so that every run starts from the same cache state.
      if (cuttHipMemsetAsync(odata, 0xFF, numBytes, (void*)stream) != 0 ||
          cuttHipDeviceSynchronize() != 0 || cuttHipEventRecord(evStart, (void*)stream) != 0 ||
          p.launch(idata, odata) != 0 || cuttHipEventRecord(evStop, (void*)stream) != 0 ||
          cuttHipEventSynchronize(evStop) != 0)
        return false;
      float ms = 0;
      if (cuttHipEventElapsedMs(evStart, evStop, &ms) != 0) return false;
      t = std::min(t, (double)ms * 1e3);
      if (t > 3.0 * bestUs) break;  // hopeless: do not spend a second run on it
    }
    return true;
  };

  std::vector<double> us(plans.size(), 0.0);
  int best = -1;
  for (int i = 0; i < (int)plans.size() && !failed; i++) {
    Plan& p = plans[i];
    if (p.method != kTrivial && p.model.usPredicted > margin * bestPred) continue;
    double t;
    if (!timePlan(p, t)) { failed = true; break; }
    us[i] = t;
    if (t < bestUs) {
      bestUs = t;
      if (best >= 0) plans[best].release();
      best = i;
    } else {
      p.release();
    }
  }
  // Second stage: the winner's launch geometry is tuned one knob at a time (tile order, work items
  // per workgroup, order of the Mbar ranks, cache policy); a setting that measures faster is kept
  // for the knobs that follow.
  if (!failed && best >= 0 && plans[best].method != kTrivial) {
    const bool tiled = plans[best].method == kTiled || plans[best].method == kTiledCopy;
    // options that reproduce the winner as it stands
    PlannerOptions cur = plannerOptions(force);
    cur.cachePolicy = cachePolicyOf(plans[best]);
    if (tiled) {
      const bool t = plans[best].method == kTiled;
      cur.tiledOrder = t ? plans[best].tiled.order : plans[best].tcopy.order;
      cur.superM = (int)(t ? plans[best].tiled.superM : plans[best].tcopy.superM);
      cur.superK = (int)(t ? plans[best].tiled.superK : plans[best].tcopy.superK);
      cur.superAuto = false;
      if (cur.tiledOrder == 7) {  // a free numbering is reproduced from its digits
        cur.tileDigits = formatTileDigits(t ? plans[best].tiled.digits : plans[best].tcopy.digits);
        cur.tiledOrder = -1;
      }
    } else {
      cur.maxItemsPerBlock = plans[best].packed.itemsPerBlock;
      cur.itemOrder = plans[best].packed.itemOrder;
      // (a winner whose work items are numbered by address bits keeps that through the variants: the order is
      // left to the planner again, which re-derives the numbering for the variant's geometry)
      if (plans[best].itemDigits.n > 0) cur.itemOrder = -1;
    }
    if (plans[best].method == kTiled) {
      cur.tiledGrouped = plans[best].tiled.grouped;
      cur.tiledAligned = plans[best].tiled.alignedStores;
    }
    const PlannerOptions start = cur;

    // Tries `v`; keeps it (and returns true) if it is faster than the best so far.
    auto tryVariant = [&](const PlannerOptions& v, bool sameGridIsSamePlan) -> bool {
      Plan q;
      if (!rebuildPlan(plans[best], props, v, q)) return false;
      if (sameGridIsSamePlan && q.numBlocks == plans[best].numBlocks) return false;
      setCachePolicy(q, v.cachePolicy);
      if (!estimatePlan(q, props, 10)) return false;
      double t;
      if (!timePlan(q, t)) { failed = true; return false; }
      if (t >= bestUs) return false;
      bestUs = t;
      us.push_back(t);
      plans[best].release();
      plans.push_back(std::move(q));
      best = (int)plans.size() - 1;
      return true;
    };

    if (tiled) {
      // patches of several shapes instead of strips (small patches walked for all Mbar positions in
      // turn make long sequential streams of a batched 2-D transpose: C2 +4...7 %), rows of tiles
      // along Mm / along Mk, strips per Mbar position / for all Mbar positions in turn
      struct TileKnob { int order, superM, superK; };
      for (const TileKnob& k : {TileKnob{5, 16, 16}, TileKnob{5, 2, 8}, TileKnob{5, 8, 2}, TileKnob{5, 32, 2},
                                TileKnob{5, 4, 8}, TileKnob{5, 8, 8}, TileKnob{5, 8, 4096}, TileKnob{5, 4, 4096},
                                TileKnob{1, 8, 4096}, TileKnob{2, 8, 4096}, TileKnob{3, 8, 4096},
                                TileKnob{3, 16, 16},
                                // small patches in order 6 (batched transposes of power-of-two sizes: up to +15 %)
                                TileKnob{6, 2, 2}, TileKnob{6, 1, 1}, TileKnob{6, 2, 1}, TileKnob{6, 1, 2},
                                TileKnob{6, 2, 4}, TileKnob{6, 4, 2}, TileKnob{6, 4, 4}, TileKnob{6, 1, 4}}) {
        if (failed) break;
        if (k.order == 6 && plans[best].split.volMbar <= 1) continue;
        if (k.order == start.tiledOrder && k.superM == start.superM && k.superK == start.superK) continue;
        PlannerOptions v = cur;
        v.tiledOrder = k.order; v.superM = k.superM; v.superK = k.superK;
        v.tileDigits.clear();
        if (tryVariant(v, false)) cur = v;
      }
      // sixteen or four rows per lane in flight
      if (!failed && plans[best].method == kTiled && !std::getenv("CUTT_TILED_GROUPED")) {
        PlannerOptions v = cur;
        v.tiledGrouped = 1 - cur.tiledGrouped;
        if (tryVariant(v, false)) cur = v;
      }
      // every tile row storing its own line-aligned window (measured: +2...+4 % on some 8-byte
      // tensors with output runs off the 128-byte grid, -5...-15 % on others, so only by trial)
      if (!failed && plans[best].method == kTiled && !std::getenv("CUTT_TILED_ALIGNED") &&
          ((int64_t)plans[best].tiled.volMk * plans[best].pb.elemSize % 128 != 0 ||
           (int64_t)plans[best].tiled.strideOutM * plans[best].pb.elemSize % 128 != 0)) {
        PlannerOptions v = cur;
        v.tiledAligned = 1;
        v.tiledGrouped = 0;
        if (tryVariant(v, false)) cur = v;
      }
    } else {
      for (int ipb : {1, 2, 4, 8}) {
        if (failed) break;
        if (ipb == start.maxItemsPerBlock) continue;
        PlannerOptions v = cur;
        v.maxItemsPerBlock = ipb;
        if (tryVariant(v, true)) cur = v;
      }
      // which items a workgroup takes: neighbouring slabs, its own slabs at several Mbar positions,
      // or every B-th item of its XCD's chunk
      for (int order : {0, 1, 2}) {
        if (failed || std::getenv("CUTT_ITEM_ORDER")) break;
        if (order == start.itemOrder) continue;
        PlannerOptions v = cur;
        v.itemOrder = order;
        Plan probe;
        if (!rebuildPlan(plans[best], props, v, probe) || probe.packed.itemOrder != order) continue;  // falls back to another order
        if (tryVariant(v, false)) cur = v;
      }
    }
    // the order in which consecutive work items (or strips of tiles) walk the Mbar ranks decides
    // which partly used lines neighbouring workgroups share in the L2; it can move the time by 20 %
    for (int order : {0, 1, 2}) {
      if (failed || std::getenv("CUTT_MBAR_ORDER")) break;
      if (order == start.mbarOrder) continue;
      PlannerOptions v = cur;
      v.mbarOrder = order;
      if (tryVariant(v, false)) cur = v;
    }
    // workgroup b at logical position b (the XCDs then interleave instead of walking a chunk each):
    // rarely better, but then by 5-10 % (measured on PackedSplit plans with long runs)
    if (!failed && !std::getenv("CUTT_XCD_AWARE") && cur.xcdAware) {
      PlannerOptions v = cur;
      v.xcdAware = false;
      if (tryVariant(v, false)) cur = v;
    }
    // ... and the other cache policies of the global accesses
    for (int pol : {0, 1, 3}) {
      if (failed || std::getenv("CUTT_CACHE_POLICY")) break;
      if (pol == start.cachePolicy) continue;
      PlannerOptions v = cur;
      v.cachePolicy = pol;
      if (tryVariant(v, false)) cur = v;
    }
  }
  if (failed || best < 0) return CUTT_INTERNAL_ERROR;

  // Play-off against the plan cuttPlan would return.  The winner is the best of up to a hundred timings of two
  // runs each, so its own time is an optimistic one; the heuristic plan (the model's pick with its Mbar order
  // and cache policy refined) is not among the candidates as such.  Both are timed again in turn and the
  // faster one is kept, so that the measuring planner does not end behind the heuristic one by more than the
  // noise of these last runs.
  if (plans[best].method != kTrivial && !std::getenv("CUTT_MEASURE_NO_PLAYOFF")) {
    std::vector<Plan> again;
    if (createPlans(orig, red, props, plannerOptions(force), again) && !again.empty() && estimateAll(again, props)) {
      refineMbarOrder(again, props, force);
      const int h = chooseHeuristic(again);
      if (h >= 0 && again[h].method != kTrivial) {
        chooseCachePolicy(again[h], props);
        Plan heur = std::move(again[h]);
        double tw = 1e300, th = 1e300;
        for (int round = 0; round < 2 && !failed; round++) {
          double t;
          if (!timePlan(heur, t)) { failed = true; break; }
          th = std::min(th, t);
          if (!timePlan(plans[best], t)) { failed = true; break; }
          tw = std::min(tw, t);
        }
        if (failed) return CUTT_INTERNAL_ERROR;
        if (th < tw) {
          plans[best].release();
          us.push_back(th);
          plans.push_back(std::move(heur));
          best = (int)plans.size() - 1;
          bestUs = th;
        } else {
          heur.release();
          bestUs = tw;
        }
      }
    }
  }

  {
    std::lock_guard<std::mutex> lock(gMutex);
    gLastMeasurement.resize(plans.size());
    for (size_t i = 0; i < plans.size(); i++) {
      fillInfo(plans[i], gLastMeasurement[i]);
      gLastMeasurement[i].usMeasured = us[i];
      gLastMeasurement[i].numCandidates = (int)plans.size();
    }
  }
  out.numCandidates = (int)plans.size();
  out.bestUs = bestUs;
  out.plan = std::move(plans[best]);
  return CUTT_SUCCESS;
}

static cuttResult planFromCandidateImpl(cuttHandle* handle, int rank, int* dim, int* permutation,
                                        size_t sizeofType, hipStream_t stream, int index) {
  const auto t0 = std::chrono::steady_clock::now();
  if (!handle) return CUTT_INVALID_PARAMETER;
  cuttResult chk = checkInput(rank, dim, permutation, sizeofType);
  if (chk != CUTT_SUCCESS) return chk;
  int deviceID;
  cuttHipDeviceProps props;
  if (!currentDevice(deviceID, props)) return CUTT_INTERNAL_ERROR;
  int force;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    force = methodOverrideLocked();
  }
  std::vector<Plan> plans;
  if (!enumerate(rank, dim, permutation, sizeofType, props, force, plans)) return CUTT_INTERNAL_ERROR;
  if (index < 0 || index >= (int)plans.size()) return CUTT_INVALID_PARAMETER;
  if (!estimateAndTune(plans[index], props)) return CUTT_INTERNAL_ERROR;
  return storePlan(handle, std::move(plans[index]), (void*)stream, deviceID, (int)plans.size(), 0.0, t0);
}

// The C entry points that plan: nothing a planner throws (std::bad_alloc from its tables) may
// cross the C boundary; the caller gets CUTT_INTERNAL_ERROR instead.
extern "C" cuttResult cuttPlan(cuttHandle* handle, int rank, int* dim, int* permutation,
                               size_t sizeofType, hipStream_t stream) {
  try {
    return planImpl(handle, rank, dim, permutation, sizeofType, stream);
  } catch (...) {
    return CUTT_INTERNAL_ERROR;
  }
}

extern "C" cuttResult cuttExecuteNoAlloc(int rank, int* dim, int* permutation, size_t sizeofType,
                                         hipStream_t stream, void* idata, void* odata) {
  try {
    return executeNoAllocImpl(rank, dim, permutation, sizeofType, stream, idata, odata);
  } catch (...) {
    return CUTT_INTERNAL_ERROR;
  }
}

extern "C" cuttResult cuttPlanMeasure(cuttHandle* handle, int rank, int* dim, int* permutation,
                                      size_t sizeofType, hipStream_t stream, void* idata, void* odata) {
  try {
    return planMeasureImpl(handle, rank, dim, permutation, sizeofType, stream, idata, odata);
  } catch (...) {
    return CUTT_INTERNAL_ERROR;
  }
}

extern "C" cuttResult cuttPlanFromCandidate(cuttHandle* handle, int rank, int* dim, int* permutation,
                                            size_t sizeofType, hipStream_t stream, int index) {
  try {
    return planFromCandidateImpl(handle, rank, dim, permutation, sizeofType, stream, index);
  } catch (...) {
    return CUTT_INTERNAL_ERROR;
  }
}

extern "C" cuttResult cuttDestroy(cuttHandle handle) {
  std::shared_ptr<StoredPlan> sp;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    auto it = gPlans.find(handle);
    if (it == gPlans.end()) return CUTT_INVALID_PLAN;
    sp = std::move(it->second);
    gPlans.erase(it);
  }
  sp.reset();  // frees the plan outside the lock, unless a cuttExecute still holds it
  return CUTT_SUCCESS;
}

extern "C" cuttResult cuttExecute(cuttHandle handle, void* idata, void* odata) {
  std::shared_ptr<StoredPlan> sp;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    auto it = gPlans.find(handle);
    if (it == gPlans.end()) return CUTT_INVALID_PLAN;
    sp = it->second;
  }
  if (idata == odata || !idata || !odata) return CUTT_INVALID_PARAMETER;
  int deviceID;
  if (cuttHipGetDevice(&deviceID) != 0) return CUTT_INTERNAL_ERROR;
  if (deviceID != sp->plan.deviceID) return CUTT_INVALID_DEVICE;
  if (sp->pieces.empty()) {
    if (sp->plan.launch(idata, odata) != 0) return CUTT_INTERNAL_ERROR;
    return CUTT_SUCCESS;
  }
  // a tensor in pieces: one launch per piece, all on the plan's stream
  const int64_t es = sp->plan.pb.elemSize;
  for (const SlabPiece& piece : sp->pieces) {
    Plan& p = piece.shape == 0 ? sp->plan : sp->more[piece.shape - 1];
    if (p.launch((const char*)idata + piece.baseIn * es, (char*)odata + piece.baseOut * es) != 0)
      return CUTT_INTERNAL_ERROR;
  }
  return CUTT_SUCCESS;
}

// ---------------------------------------------------------------------------
// cutt_ext.h
// ---------------------------------------------------------------------------
extern "C" cuttResult cuttGetPlanInfo(cuttHandle handle, cuttPlanInfo* info) {
  if (!info) return CUTT_INVALID_PARAMETER;
  std::lock_guard<std::mutex> lock(gMutex);
  auto it = gPlans.find(handle);
  if (it == gPlans.end()) return CUTT_INVALID_PLAN;
  fillInfo(it->second->plan, *info);
  if (!it->second->pieces.empty()) {
    info->numPieces = (int)it->second->pieces.size();
    info->numShapes = 1 + (int)it->second->more.size();
  }
  info->numCandidates = it->second->numCandidates;
  info->planMs = it->second->planMs;
  info->usMeasured = it->second->usMeasured;
  return CUTT_SUCCESS;
}

extern "C" cuttResult cuttCountAddressStream(cuttHandle handle, int numSamples, cuttStreamCounts* onDevice,
                                             cuttStreamCounts* byModel) {
  if (!onDevice || !byModel || numSamples < 0) return CUTT_INVALID_PARAMETER;
  std::shared_ptr<StoredPlan> sp;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    auto it = gPlans.find(handle);
    if (it == gPlans.end()) return CUTT_INVALID_PLAN;
    sp = it->second;
  }
  Plan& p = sp->plan;
  if (p.method == kTrivial) return CUTT_INVALID_PARAMETER;
  try {
    cuttHipStreamCounts d;
    std::memset(&d, 0, sizeof(d));
    int rc;
    if (p.method == kTiled) rc = cuttHipCountTiled(&p.tiled, &d, p.stream);
    else if (p.method == kTiledCopy) rc = cuttHipCountTiledCopy(&p.tcopy, &d, p.stream);
    else rc = cuttHipCountPacked(&p.packed, &d, p.stream);
    if (rc != 0) return CUTT_INTERNAL_ERROR;
    *onDevice = cuttStreamCounts{(double)d.rdInstr, (double)d.wrInstr, (double)d.rdInstrIdle, (double)d.wrInstrIdle,
                                 (double)d.rdLines, (double)d.wrLines, (double)d.rdSectors, (double)d.wrSectors,
                                 (double)d.wrPartialLines, (double)d.ldsCycles, (int)d.ldsMaxDegree};
    // the host model's walk over a copy of the plan (the plan itself keeps its estimate)
    Plan q = p.clone();
    int deviceID;
    cuttHipDeviceProps props;
    if (!currentDevice(deviceID, props)) return CUTT_INTERNAL_ERROR;
    if (!estimatePlan(q, props, numSamples)) return CUTT_INTERNAL_ERROR;
    *byModel = cuttStreamCounts{q.model.rdInstr, q.model.wrInstr, 0.0, 0.0, q.model.rdLines, q.model.wrLines,
                                q.model.rdSectors, q.model.wrSectors, q.model.wrPartialLines, q.model.ldsCycles, 0};
  } catch (...) {
    return CUTT_INTERNAL_ERROR;
  }
  return CUTT_SUCCESS;
}

extern "C" void cuttSetMethodOverride(int method) {
  std::lock_guard<std::mutex> lock(gMutex);
  gMethodOverride = (method > 0 && method < kNumMethods) ? method : 0;
}

extern "C" int cuttGetMethodOverride(void) {
  std::lock_guard<std::mutex> lock(gMutex);
  return methodOverrideLocked();
}

extern "C" int cuttGetLastMeasurement(cuttPlanInfo* infos, int maxInfos) {
  try {
    std::lock_guard<std::mutex> lock(gMutex);
    const int n = (int)gLastMeasurement.size();
    for (int i = 0; i < n && i < maxInfos && infos; i++) infos[i] = gLastMeasurement[i];
    return n;
  } catch (...) {  // nothing may cross the C boundary
    return -1;
  }
}

extern "C" int cuttReduceRanks(int rank, const int* dim, const int* permutation, int* redDim,
                               int* redPermutation) {
  try {
    if (rank < 1 || !dim || !permutation || !redDim || !redPermutation) return -1;
    std::vector<int> d, p;
    reduceRanks(rank, dim, permutation, d, p);
    for (size_t i = 0; i < d.size(); i++) {
      redDim[i] = d[i];
      redPermutation[i] = p[i];
    }
    return (int)d.size();
  } catch (...) {  // nothing may cross the C boundary
    return -1;
  }
}

namespace {
struct CandidateList {
  std::vector<Plan> plans;
  int best = -1;
};
}  // namespace

extern "C" void cuttDeviceCallCounts(unsigned long long* allocations, unsigned long long* uploads) {
  cuttHipCallCounts(allocations, uploads);
}

extern "C" void cuttClearPlanCache(void) {
  std::lock_guard<std::mutex> lock(gMutex);
  gDecisionIndex.clear();
  gDecisions.clear();
}

extern "C" void* cuttCandidatesCreateEx(int rank, const int* dim, const int* permutation,
                                        size_t sizeofType, size_t ldsPerBlock) {
  try {
    if (checkInput(rank, dim, permutation, sizeofType) != CUTT_SUCCESS) return nullptr;
    int force;
    {
      std::lock_guard<std::mutex> lock(gMutex);
      force = methodOverrideLocked();
    }
    std::unique_ptr<CandidateList> l(new CandidateList());
    cuttHipDeviceProps props = defaultMI355XProps();
    if (ldsPerBlock) props.ldsPerBlock = props.ldsPerCU = ldsPerBlock;
    if (!enumerate(rank, dim, permutation, sizeofType, props, force, l->plans)) return nullptr;
    if (!estimateAll(l->plans, props)) return nullptr;
    l->best = chooseHeuristic(l->plans);
    return l.release();
  } catch (...) {  // nothing may cross the C boundary
    return nullptr;
  }
}

extern "C" void* cuttCandidatesCreateStrided(int rank, const int* dim, const int* permutation, size_t sizeofType,
                                             const long long* strideIn, const long long* strideOut,
                                             size_t ldsPerBlock) {
  try {
    if (checkInput(rank, dim, permutation, sizeofType) != CUTT_SUCCESS || !strideIn || !strideOut) return nullptr;
    int force;
    {
      std::lock_guard<std::mutex> lock(gMutex);
      force = methodOverrideLocked();
    }
    std::vector<int64_t> sIn(strideIn, strideIn + rank), sOut(strideOut, strideOut + rank);
    Problem pb;
    if (!pb.setStrided(rank, dim, permutation, (int)sizeofType, sIn.data(), sOut.data())) return nullptr;
    std::unique_ptr<CandidateList> l(new CandidateList());
    cuttHipDeviceProps props = defaultMI355XProps();
    if (ldsPerBlock) props.ldsPerBlock = props.ldsPerCU = ldsPerBlock;
    if (!createPlans(pb, pb, props, plannerOptions(force), l->plans) || !estimateAll(l->plans, props)) return nullptr;
    l->best = chooseHeuristic(l->plans);
    return l.release();
  } catch (...) {  // nothing may cross the C boundary
    return nullptr;
  }
}

extern "C" long long cuttSlabDecomposition(int rank, const int* dim, const int* permutation, size_t sizeofType,
                                           long long spanLimit, long long* values, long long maxCount) {
  try {
    bool large = false;
    if (checkInput(rank, dim, permutation, sizeofType, &large) != CUTT_SUCCESS) return -1;
    std::vector<int> redDim, redPerm;
    reduceRanks(rank, dim, permutation, redDim, redPerm);
    SlabDecomposition dec;
    if (!slabDecompose((int)redDim.size(), redDim.data(), redPerm.data(), (int)sizeofType,
                       spanLimit > 0 ? spanLimit : slabSpanLimit(), dec))
      return -1;
    std::vector<long long> v = {(long long)dec.shapes.size(), (long long)dec.pieces.size()};
    for (const Problem& p : dec.shapes) {
      v.push_back(p.rank);
      for (int r = 0; r < p.rank; r++) v.push_back(p.dim[r]);
      for (int r = 0; r < p.rank; r++) v.push_back(p.perm[r]);
      for (int r = 0; r < p.rank; r++) v.push_back(p.strideIn[r]);
      for (int r = 0; r < p.rank; r++) v.push_back(p.strideOut[r]);
    }
    for (const SlabPiece& q : dec.pieces) {
      v.push_back(q.shape);
      v.push_back(q.baseIn);
      v.push_back(q.baseOut);
    }
    if (values)
      for (long long i = 0; i < std::min<long long>(maxCount, (long long)v.size()); i++) values[i] = v[i];
    return (long long)v.size();
  } catch (...) {  // nothing may cross the C boundary
    return -1;
  }
}

extern "C" void* cuttCandidatesCreate(int rank, const int* dim, const int* permutation,
                                      size_t sizeofType) {
  return cuttCandidatesCreateEx(rank, dim, permutation, sizeofType, 0);
}

extern "C" void cuttCandidatesFree(void* list) { delete (CandidateList*)list; }
extern "C" int cuttCandidatesCount(void* list) { return list ? (int)((CandidateList*)list)->plans.size() : -1; }
extern "C" int cuttCandidatesBest(void* list) { return list ? ((CandidateList*)list)->best : -1; }

extern "C" int cuttCandidatesInfo(void* list, int index, cuttPlanInfo* info) {
  CandidateList* l = (CandidateList*)list;
  if (!l || !info || index < 0 || index >= (int)l->plans.size()) return -1;
  fillInfo(l->plans[index], *info);
  info->numCandidates = (int)l->plans.size();
  return 0;
}

extern "C" long long cuttCandidatesData(void* list, int index, int what, int cls, long long* values,
                                        long long maxCount) {
  try {
    CandidateList* l = (CandidateList*)list;
    if (!l || index < 0 || index >= (int)l->plans.size() || cls < 0 || cls > 3) return -1;
    const Plan& p = l->plans[index];
    std::vector<long long> v;
    const bool packed = p.method == kPacked || p.method == kPackedSplit;
    switch (what) {
      case 0: {
        const cuttHipMbar& mb = packed ? p.packed.mbar : (p.method == kTiled ? p.tiled.mbar : p.tcopy.mbar);
        if (p.method == kTrivial) break;
        for (int k = 0; k < mb.n; k++) {
          v.push_back(mb.d[k].extent);
          v.push_back(mb.d[k].strideIn);
          v.push_back(mb.d[k].strideOut);
        }
      } break;
      case 1:
        if (p.method == kTiled)
          v = {p.tiled.volMm, p.tiled.volMk, p.tiled.strideInK, p.tiled.strideOutM, p.tiled.tilesM,
               p.tiled.tilesK, p.tiled.volMbar, p.tiled.order, p.tiled.xcdChunk, p.tiled.superM, p.tiled.superK};
        else if (p.method == kTiledCopy)
          v = {p.tcopy.volMm, p.tcopy.volMk, p.tcopy.strideInK, p.tcopy.strideOutK, p.tcopy.tilesM,
               p.tcopy.tilesK, p.tcopy.volMbar, p.tcopy.order, p.tcopy.xcdChunk, p.tcopy.superM, p.tcopy.superK};
        else
          return -1;
        break;
      case 2:
        if (!packed) return -1;
        v = {p.packed.numThreads, p.packed.volMbar, p.packed.itemsPerBlock, p.packed.padShift,
             p.packed.ldsElems, p.packed.xcdChunk, p.packed.elemsPerThread, p.packed.itemOrder};
        for (int i = 0; i < 2; i++) {
          const cuttHipSplitRank& sr = p.packed.split[i];
          v.insert(v.end(), {sr.numSplit, sr.slabFloor, sr.slabRem, sr.strideIn, sr.strideOut});
        }
        break;
      case 3: {
        if (!packed) return -1;
        const cuttHipPackedClass& k = p.packed.cls[cls];
        v = {k.vol, k.inCont, k.outCont};
      } break;
      case 4:
        if (!packed) return -1;
        v.assign(p.tab[cls].rowIn.begin(), p.tab[cls].rowIn.end());
        break;
      case 5:
        if (!packed) return -1;
        v.assign(p.tab[cls].rowOut.begin(), p.tab[cls].rowOut.end());
        break;
      case 6:
        if (!packed) return -1;
        v.assign(p.tab[cls].shIdx.begin(), p.tab[cls].shIdx.end());
        break;
      case 7:  // Tiled: (extent, stride) of the ranks a tile axis runs over: cls 0 = Mk (input strides), 1 = Mm (output strides)
        if (p.method != kTiled || cls > 1) return -1;
        {
          const cuttHipRowRadix& rr = cls == 0 ? p.tiled.rowsK : p.tiled.rowsM;
          for (int k = 0; k < rr.n; k++) {
            v.push_back(rr.extent[k]);
            v.push_back(rr.stride[k]);
          }
        }
        break;
      case 8:  // tile order 7 / work-item order 3: (coordinate, radix, weight) of the digits, fastest first
        if (p.method != kTiled && p.method != kTiledCopy && !packed) return -1;
        {
          const cuttHipTileDigits& dg = packed ? p.itemDigits : (p.method == kTiled ? p.tiled.digits : p.tcopy.digits);
          for (int k = 0; k < dg.n; k++) {
            v.push_back(dg.d[k].which);
            v.push_back(dg.d[k].radix);
            v.push_back(dg.d[k].weight);
          }
        }
        break;
      case 9:  // Tiled / TiledCopy, tile order 7: the digits as the kernels decode them lane-parallel: lanes (0/1), total,
               // then per digit radix, stepM, stepK, strideIn, strideOut
        if (p.method != kTiled && p.method != kTiledCopy) return -1;
        {
          const cuttHipTileDigits& dg = p.method == kTiled ? p.tiled.digits : p.tcopy.digits;
          v.push_back(dg.lanes);
          v.push_back(dg.total);
          for (int k = 0; k < dg.n && dg.lanes; k++)
            v.insert(v.end(), {dg.lane[k].radix, dg.lane[k].stepM, dg.lane[k].stepK, dg.lane[k].strideIn, dg.lane[k].strideOut});
        }
        break;
      default:
        return -1;
    }
    for (long long i = 0; i < (long long)v.size() && i < maxCount && values; i++) values[i] = v[(size_t)i];
    return (long long)v.size();
  } catch (...) {  // nothing may cross the C boundary
    return -1;
  }
}

extern "C" int cuttModelGlTransactionsSeg(const int* seg, int n) { return glTransactions(seg, n); }
extern "C" int cuttModelGlTransactionsCont(int pos, int n, int accWidth) {
  return glTransactions(pos, n, accWidth);
}
extern "C" void cuttModelCacheLinesSeg(const int* seg, int n, int cacheWidth, int* clFull, int* clPart) {
  countCacheLines(seg, n, cacheWidth, *clFull, *clPart);
}
extern "C" void cuttModelCacheLinesCont(int pos, int n, int cacheWidth, int* clFull, int* clPart) {
  countCacheLines(pos, n, cacheWidth, *clFull, *clPart);
}
extern "C" void cuttModelShTransactions(int waveSize, int numBanks, int numThreads, int volMmk,
                                        const int* msh, int numMsh, int* out4) {
  std::vector<ShConv> m(numMsh);
  for (int i = 0; i < numMsh; i++) m[i] = {msh[3 * i], msh[3 * i + 1], msh[3 * i + 2]};
  out4[0] = out4[1] = out4[2] = out4[3] = 0;
  countShTransactions(waveSize, numBanks, numThreads, volMmk, m.data(), numMsh, out4[0], out4[1],
                      out4[2], out4[3]);
}
