/*
 * plan.h - host-side planner: rank fusing, index-set splits, candidate
 * enumeration, index tables and launch geometry.  Pure host C++; the device is
 * reached only through hip_layer.h.
 *
 * Counterpart of reference src/cuttplan.h:36-212 (method enum, TensorSplit,
 * LaunchConfig, cuttPlan_t) with a different organisation: a candidate owns
 * the ready-to-launch kernel arguments, and Packed tables are compact
 * (one offset per contiguous row + a 16-bit LDS gather index per element).
 */
#ifndef CUTT_PLAN_H
#define CUTT_PLAN_H

#include <cstdint>
#include <string>
#include <vector>

#include "hip_layer.h"

namespace cutt {

// Same numbering as the reference's method enum (src/cuttplan.h:37-39).
enum Method { kUnknown = 0, kTrivial = 1, kPacked = 2, kPackedSplit = 3, kTiled = 4, kTiledCopy = 5, kNumMethods };

const char* methodName(int method);

// A transpose problem: dims (dim[0] fastest), permutation, element size, strides.
// Usually both tensors are dense (strides follow from the extents).  A piece of a larger tensor
// (slab.h) keeps the larger tensor's strides: then a rank may not continue where the previous one
// ends, which gapIn / gapOut record, and only ranks without a gap between them form contiguous runs.
struct Problem {
  int rank = 0;
  int elemSize = 0;
  std::vector<int> dim;
  std::vector<int> perm;       // output rank j is input rank perm[j]
  std::vector<int> inv;        // inv[perm[j]] = j
  std::vector<int64_t> strideIn;   // input stride of input rank r
  std::vector<int64_t> strideOut;  // output stride of input rank r
  std::vector<char> gapIn;     // gapIn[r]: input rank r+1 does not start where rank r ends
  std::vector<char> gapOut;    // gapOut[r]: the rank that follows r in the output does not start where r ends
  bool dense = true;           // no gaps and unit strides of the two leading ranks
  int64_t volume = 0;
  int64_t span = 0;            // elements from the first to the last one, on the wider side (= volume when dense)

  void set(int rank, const int* dim, const int* perm, int elemSize);
  // Same with given strides; false unless the leading rank of each side has stride 1.
  bool setStrided(int rank, const int* dim, const int* perm, int elemSize, const int64_t* strideIn,
                  const int64_t* strideOut);
};

// Fuse runs of ranks that stay adjacent and in order (reference src/cuttplan.cpp:63-126).
void reduceRanks(int rank, const int* dim, const int* perm, std::vector<int>& redDim,
                 std::vector<int>& redPerm);

/*
 * How a candidate divides the ranks (vocabulary of reference src/cuttplan.h:41-82):
 *   Mm   = the first numMm input ranks,  Mk = the first numMk output ranks,
 *   Mmk  = Mm u Mk (staged by one workgroup), Mbar = everything else.
 */
struct Split {
  int method = kUnknown;
  int numMm = 0, numMk = 0;
  int sizeMmk = 0, sizeMbar = 0, sizeMkBar = 0;
  int64_t volMm = 0, volMk = 0, volMmk = 0, volMkBar = 0, volMbar = 0;
  int64_t volMmkInCont = 0, volMmkOutCont = 0;  // for the largest slab when split
  // PackedSplit: up to two ranks of Mmk are cut into slabs (slot 0 first; an unused slot has
  // splitRank -1 and numSplit 1)
  int splitRank[2] = {-1, -1};
  int splitDim[2] = {0, 0};
  int numSplit[2] = {1, 1};
  int64_t volMmkUnsplit = 0;
  std::vector<char> inMmk;  // per input rank

  void update(int numMm, int numMk, const Problem& pb);
  int slabMax(int i) const { return splitRank[i] < 0 ? 1 : (splitDim[i] + numSplit[i] - 1) / numSplit[i]; }
  int splitSlot(int rank) const { return rank == splitRank[0] ? 0 : (rank == splitRank[1] ? 1 : -1); }
  int64_t volStaged() const;  // elements one workgroup stages at most
};

// Host copy of the index tables of one slab-size class (see cuttHipPackedClass): one offset per
// contiguous run on the input and on the output side, and the LDS gather index per element.
struct PackedTables {
  int vol = 0, inCont = 0, outCont = 0;
  std::vector<uint32_t> rowIn, rowOut;
  std::vector<uint16_t> shIdx;
};

// Counters and estimate produced by the cost model (model.h).
struct ModelResult {
  double rdLines = 0, wrLines = 0;     // 128-byte lines touched, whole tensor
  double rdInstr = 0, wrInstr = 0;     // wavefront-level memory instructions, whole tensor
  double wrPartialLines = 0;           // written lines not fully covered by one workgroup
  double rdSectors = 0, wrSectors = 0; // 32-byte sectors touched
  double ldsCycles = 0;                // LDS cycles incl. bank conflicts, whole tensor
  double blocksPerCU = 0;
  // Work items between the two workgroups that touch the two sides of a run's end (the next run
  // in memory): small = the shared line is still in the L2 when its other part is accessed.
  double rdEdgeDist = 0, wrEdgeDist = 0;
  // Tiled over fused rank sets: the output runs of a tile row end where the Mk set ends, and the run that
  // follows in memory may belong to another row of the Mm axis, many tiles away: its distance, and the share
  // of the partly written lines that lie at such run ends (the others lie between two tiles along Mk).
  double wrEdgeOuter = 0, wrOuterShare = 0;
  double usPredicted = 0;              // predicted time in microseconds (ranking key)
};

struct Plan {
  int method = kUnknown;
  Split split;
  Problem pb;             // the problem this candidate was built from (original or fused)
  bool fromReduced = false;
  int deviceID = -1;
  void* stream = nullptr;

  cuttHipTiledArgs tiled;
  cuttHipTiledCopyArgs tcopy;
  cuttHipPackedArgs packed;
  cuttHipTileDigits itemDigits;  // Packed/PackedSplit: n > 0 if the work items are numbered by these digits (setupPacked)
  size_t ldsBytes = 0;
  int64_t numBlocks = 0;
  int numThreads = 0;

  // Packed host tables, built on demand (buildTables) and device copies (activate).
  PackedTables tab[4];
  bool tablesBuilt = false;
  void* dTables = nullptr;
  bool launchable = false;  // set by activate(): the launch arguments passed their check

  ModelResult model;

  Plan();
  ~Plan();
  Plan(const Plan&) = delete;
  Plan& operator=(const Plan&) = delete;
  Plan(Plan&& o) noexcept;
  Plan& operator=(Plan&& o) noexcept;

  Plan clone() const;             // host-side copy of a plan that has no device tables yet
  bool buildTables();             // Packed/PackedSplit: fill tab[]; others: no-op
  int activate();                 // upload tables, check the launch arguments; 0 or an error code
  // Like activate(), but the tables are built by a kernel on `stream` in device memory the caller
  // provides (`capacity` bytes, 16-byte aligned) instead of being allocated and uploaded; the plan
  // does not own that memory.  Nothing is allocated on the device.
  int activateInPlace(void* tables, size_t capacity);
  size_t tableBytes() const;      // device bytes of the index tables (0 for methods without)
  int launch(const void* in, void* out);  // asynchronous on stream
  void release();                 // free device tables
  std::string describe() const;
};

struct PlannerOptions {
  int forceMethod = 0;      // 0 = all methods, else only this Method (Trivial always allowed)
  int tiledOrder = -1;      // -1 = planner's choice (super-tiles)
  int superM = 8, superK = 4096;  // super-tile shape for tiled orders 3-6: strips of 8 tiles along Mm
  bool superAuto = true;    // the planner may replace that shape where it measured a better one (see tiledBlocks)
  std::string tileDigits;   // non-empty: tiled order 7 with this mixed-radix numbering, fastest digit first, e.g.
                            // "m2,k8,b0,m0,k0" (m / k = tile along Mm / Mk, b = Mbar position; radix 0 = what is left)
  std::string itemDigits;   // non-empty: the packed kernel's work items numbered by these digits, same syntax; m / k = slab of
                            // the first / second cut rank, b = Mbar position; applies to candidates whose slabs are all of one
                            // size and whose extents the radices multiply to exactly
  int digitLanes = -1;      // tile order 7: decode the digits lane-parallel (1), digit by digit (0), planner's choice (-1)
  bool addressBits = true;  // Tiled: number the workgroups by the address bits their digits move where that rule applies (addressBitOrder)
  int tiledFuse = -1;       // Tiled over fused rank sets: -1 = planner's choice, 0 = one rank per side only
  int tiledAligned = -1;    // Tiled: line-aligned stores, -1 = planner's choice, 0 = off, 1 = on
  int tiledGrouped = -1;    // Tiled: rows of a lane in flight, -1 = planner's choice, 0 = all 16, 1 = 4 at a time
  int elemsPerThread = 0;    // Packed/PackedSplit: 0 = planner's choice, else 1, 2, 4, 8 or 16
  int packedRounds = 0;      // > 0: size the grid for this many waves of resident workgroups
  int itemOrder = -1;        // Packed/PackedSplit work-item numbering: -1 = planner's choice, 0 = a workgroup walks
                             // neighbouring slabs, 1 = it keeps its slabs and walks Mbar positions, 2 = the
                             // workgroups of an XCD take the items of their chunk round by round
  int padShift = 0;          // Packed/PackedSplit: LDS slot(p) = p + (p >> padShift); 0 = the default (5), 31 = no padding
  int maxItemsPerBlock = 0;  // Packed/PackedSplit: work items one workgroup handles at most; 0 = by item size
  int cachePolicy = 1;      // 0 default, 1 non-temporal loads, 3 non-temporal loads and stores
  int mbarOrder = 2;        // order of the Mbar ranks: 0 = input order, 1 = output order,
                            // 2 = first input rank outside Mmk, then output order
  bool wideOffsets = false; // Packed/PackedSplit: 64-bit address arithmetic also below 4 GB (tests)
  bool xcdAware = true;     // give every XCD (private L2) a contiguous chunk of the workgroup sequence
};

// Build every candidate for the original and the fused problem
// (reference src/cuttplan.cpp:681-698).  Returns false on an internal error.
bool createPlans(const Problem& orig, const Problem& red, const cuttHipDeviceProps& props,
                 const PlannerOptions& opt, std::vector<Plan>& plans);

// Same index sets as `src`, launch geometry recomputed under different options (used by the
// measuring planner to try ordering and granularity variants of its best candidate).
bool rebuildPlan(const Plan& src, const cuttHipDeviceProps& props, const PlannerOptions& opt, Plan& out);

// Text form of a tile digit list, as PlannerOptions::tileDigits takes it.
std::string formatTileDigits(const cuttHipTileDigits& dg);

// Default device description of one MI355X, used when no GPU is present (tests, offline planning).
cuttHipDeviceProps defaultMI355XProps();
// Replace fields the runtime left at zero (or at implausible values) by those of the default.
void sanitizeDeviceProps(cuttHipDeviceProps& props);

}  // namespace cutt

#endif  // CUTT_PLAN_H
