/*
 * cutt_ext.h - introspection and test hooks beside the four plan functions of
 * cutt.h.  None of these has a counterpart in the reference's public header;
 * they expose what the reference only prints (cuttPlan_t::print,
 * src/cuttplan.cpp:792-809), what its test driver reaches through internal
 * headers (testCounters, src/cuttGpuModel.h:85; reduceRanks,
 * src/cuttplan.h:215-216), and an override that pins the method so that each
 * kernel can be measured alone.
 */
#ifndef CUTT_EXT_H
#define CUTT_EXT_H

#include "cutt.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Method numbers, as in the reference's enum (src/cuttplan.h:37-39). */
enum {
  CUTT_METHOD_UNKNOWN = 0,
  CUTT_METHOD_TRIVIAL = 1,
  CUTT_METHOD_PACKED = 2,
  CUTT_METHOD_PACKEDSPLIT = 3,
  CUTT_METHOD_TILED = 4,
  CUTT_METHOD_TILEDCOPY = 5
};

/* What a plan (or a candidate) looks like. */
typedef struct cuttPlanInfo {
  int method;
  int fromReduced;      /* 1 if built from the rank-fused problem */
  int rank;             /* rank of the problem the plan was built from */
  int numMm, numMk;
  int splitRank, splitDim, numSplit;     /* first split rank (PackedSplit), -1/0/1 if none */
  int splitRank2, splitDim2, numSplit2;  /* second split rank, -1/0/1 if none */
  long long volMm, volMk, volMmk, volMbar, volMmkInCont, volMmkOutCont, volMmkUnsplit;
  long long numBlocks;
  int numThreads;
  int itemsPerBlock;    /* Packed/PackedSplit */
  int tiledOrder;       /* Tiled/TiledCopy: numbering of the workgroups, 0-7 (hip_layer.h: cuttHipTiledArgs.order) */
  unsigned long long ldsBytes;
  /* cost model */
  double usPredicted;
  double rdLines, wrLines, rdInstr, wrInstr, wrPartialLines, rdSectors, wrSectors, ldsCycles,
      blocksPerCU;
  /* filled by cuttPlanMeasure: time of this candidate's timed run, else 0 */
  double usMeasured;
  /* planning statistics of the call that made the plan */
  int numCandidates;
  double planMs;
  int cachePolicy;      /* 0 default, 1 non-temporal loads, 3 non-temporal loads and stores */
  int elemsPerThread;   /* Packed/PackedSplit */
  /* cost model: work items between the accesses to the two parts of a line shared by neighbouring
   * runs, on the read and on the write side (0 = no such neighbour) */
  double rdEdgeDist, wrEdgeDist;
  int tiledGrouped;     /* Tiled: 1 if a lane keeps 4 instead of 16 tile rows in flight */
  int superM, superK;   /* Tiled/TiledCopy: shape of the super-tiles the workgroups walk (tiled orders 3-6) */
  int tiledAligned;     /* Tiled: 1 if every tile row stores its own line-aligned window of its output run */
  int itemOrder;        /* Packed/PackedSplit: 0 = a workgroup walks neighbouring slabs, 1 = it keeps its slabs
                           and walks Mbar positions, 2 = the workgroups of an XCD take the items of their
                           chunk round by round */
  int numPieces;        /* launches per cuttExecute: 1, or the pieces of a tensor of 2^32 elements and more
                           (the other fields then describe the plan of the first piece) */
  int numShapes;        /* different shapes among those pieces (each has a plan of its own): 1..4 */
  int wideOffsets;      /* Packed/PackedSplit: 1 if the kernel instance does 64-bit address arithmetic (the
                           tensor, or the piece of a larger one, spans 4 GB and more) */
  char tileDigits[192]; /* Tiled/TiledCopy in order 7: the digits of the workgroup number, fastest first, in the
                           syntax of CUTT_TILE_DIGITS ("m2@1,k2@1,b3@64,..." = coordinate, radix, weight);
                           Packed/PackedSplit whose work items are numbered by digits (m, k = slab of the
                           first, second cut rank; b = Mbar position): those digits; else empty */
} cuttPlanInfo;

/* Describe an existing plan. */
cuttResult cuttGetPlanInfo(cuttHandle handle, cuttPlanInfo* info);

/*
 * Restrict the planner to one method (CUTT_METHOD_*; 0 = no restriction) for
 * plans created afterwards by this process.  A transpose that fuses to a plain
 * copy still yields a Trivial plan.  If the method has no feasible candidate,
 * cuttPlan returns CUTT_INTERNAL_ERROR.  The environment variable
 * CUTT_FORCE_METHOD (tiled, tiledcopy, packed, packedsplit) sets the initial
 * value.
 */
void cuttSetMethodOverride(int method);
int cuttGetMethodOverride(void);

/*
 * cuttPlan remembers what it decided for the tensors it planned last (per
 * device, method override and tuning environment; 64 entries, least recently
 * used dropped first; CUTT_PLAN_CACHE = n changes the number, 0 switches the
 * memory off), so that planning the same tensor again skips the enumeration
 * and the cost model.  Every plan still owns its device tables and its stream.
 * cuttPlanMeasure neither reads nor fills this memory.  The call below
 * forgets all decisions.  No counterpart in the reference.
 */
void cuttClearPlanCache(void);

/*
 * How often this process has allocated device memory and uploaded index tables on the library's
 * behalf so far (every cuttPlan of a Packed / PackedSplit plan does both once).  A caller that must
 * not allocate reads them around cuttExecuteNoAlloc: they do not move.  No counterpart in the reference.
 */
void cuttDeviceCallCounts(unsigned long long* allocations, unsigned long long* uploads);

/*
 * After cuttPlanMeasure: the candidates of its most recent call in this
 * process, in enumeration order (a variant of the winner that beat it is
 * appended at the end).  usMeasured is 0 for candidates that were not timed
 * because the cost model put them more than 1.6x behind its best one
 * (CUTT_MEASURE_ALL=1 times all).  Returns the number of candidates and copies
 * up to maxInfos descriptions.
 */
int cuttGetLastMeasurement(cuttPlanInfo* infos, int maxInfos);

/*
 * Create a plan from candidate number `index` of the planner's enumeration for
 * this problem on the current device (0 <= index < numCandidates, see
 * cuttPlanInfo.numCandidates; out of range -> CUTT_INVALID_PARAMETER).  Lets a
 * test or a tuning run execute every candidate, not only the chosen one.
 */
cuttResult cuttPlanFromCandidate(cuttHandle* handle, int rank, int* dim, int* permutation,
                                 size_t sizeofType, hipStream_t stream, int index);

/* Fuse ranks that stay adjacent and ordered; returns the fused rank.
 * redDim and redPermutation must hold `rank` entries. */
int cuttReduceRanks(int rank, const int* dim, const int* permutation, int* redDim,
                    int* redPermutation);

/* ---- candidate lists without a GPU (tests, offline inspection) ----------- */

/*
 * Enumerate the candidates the planner would build for this problem on a
 * device with MI355X properties (no GPU needed, nothing is launched).
 * Returns an opaque list or NULL on invalid input; free it with
 * cuttCandidatesFree.
 */
void* cuttCandidatesCreate(int rank, const int* dim, const int* permutation, size_t sizeofType);
/* Same with a different LDS size per workgroup (0 = the device's), so that small test tensors
 * also produce PackedSplit candidates. */
void* cuttCandidatesCreateEx(int rank, const int* dim, const int* permutation, size_t sizeofType,
                             size_t ldsPerBlock);
/* The candidates for one piece of a larger tensor: extents and permutation of the piece, element
 * strides of the larger tensor (per input rank, for the input and the output side; the leading
 * rank of each side must have stride 1). */
void* cuttCandidatesCreateStrided(int rank, const int* dim, const int* permutation, size_t sizeofType,
                                  const long long* strideIn, const long long* strideOut, size_t ldsPerBlock);
void cuttCandidatesFree(void* list);
int cuttCandidatesCount(void* list);
/* Index of the candidate the cost model ranks best. */
int cuttCandidatesBest(void* list);
int cuttCandidatesInfo(void* list, int index, cuttPlanInfo* info);

/*
 * How a tensor is cut into pieces that one launch can address (every piece spans at most
 * spanLimit elements of the input and of the output; 0 = the library's limit, 2^32 - 1).  The
 * ranks are fused first.  Copies up to maxCount values into `values` and returns the number
 * there are, -1 if the tensor cannot be cut (see slab.h):
 *   numShapes, numPieces,
 *   per shape: rank, extents[rank], permutation[rank], strideIn[rank], strideOut[rank],
 *   per piece: shape, baseIn, baseOut (element offsets).
 * A tensor that needs no cutting comes back as one piece of one shape.
 */
long long cuttSlabDecomposition(int rank, const int* dim, const int* permutation, size_t sizeofType,
                                long long spanLimit, long long* values, long long maxCount);

/*
 * Raw index data of candidate `index`, for checking a plan's address stream
 * on the host.  `what` selects the array, `cls` the slab class (0..3) where it
 * applies; the function copies up to maxCount 64-bit values into `values` and
 * returns the array's length (or -1).
 *
 *   what 0: Mbar table, 3 values per rank: extent, strideIn, strideOut
 *   what 1: tile geometry: volMm, volMk, strideInK, strideOut(M or K), tilesM, tilesK, volMbar, order,
 *           xcdChunk, superM, superK
 *   what 2: packed scalars: numThreads, volMbar, itemsPerBlock, padShift, ldsElems, xcdChunk,
 *           elemsPerThread, itemOrder (0: work item w = (m*numSplit1 + s1)*numSplit0 + s0; 1: a
 *           workgroup keeps its slabs, w = ((mb*numSplit1 + s1)*numSplit0 + s0)*itemsPerBlock + mi,
 *           m = mb*itemsPerBlock + mi; 2: numbered as in 0, workgroup q of a chunk of B workgroups takes
 *           chunkStart + q, chunkStart + q + B, ...), then for each of the two split slots: numSplit, slabFloor, slabRem,
 *           strideIn, strideOut
 *   what 3: class scalars: vol, inCont, outCont
 *   what 4: rowIn[] (vol/inCont input offsets, one per contiguous run)
 *   what 5: rowOut[] (vol/outCont output offsets)   what 6: shIdx[] (vol LDS gather slots)
 *   what 7: Tiled over fused rank sets: (extent, stride) of the ranks a tile axis runs over (cls 0 = Mk, 1 = Mm)
 *   what 8: the digits of a free numbering (tile order 7, or a packed plan's work items), fastest first:
 *           (coordinate, radix, weight) each
 *   what 9: tile order 7, the same digits as the kernels decode them with one digit per lane: lanes (1 if
 *           the list allows that), the product of the radices, then per digit (radix, tiles along Mm and
 *           along Mk per unit, input and output offset per unit)
 */
long long cuttCandidatesData(void* list, int index, int what, int cls, long long* values,
                             long long maxCount);

/* ---- the address stream of a plan, counted on the device ------------------
 *
 * Kernels that take a plan's launch arguments and replay the transpose kernel's address stream
 * (same workgroup numbering, same index arithmetic, same tables, no data moved) count, with 64-lane
 * ballots, what the cost model counts on the host; the call also returns the host model's walk of
 * the same plan over numSamples sampled work items (0 = every work item, then the two must agree
 * exactly).  Counterpart of the reference's cuttGpuModelKernel (src/cuttGpuModelKernel.cu:686-782),
 * which its library never calls; here a GPU test does.
 *
 *   instructions: wavefront-wide loads / stores that carry data; "idle" ones only repeat an edge
 *   element (the kernels clamp indices instead of branching; the host model does not count them)
 *   lines, sectors: distinct 128-byte / 32-byte blocks per instruction, summed
 *   wrPartialLines: ends of output runs that do not fall on a line boundary
 *   ldsCycles: Packed/PackedSplit, per gather instruction conflict degree * words + words
 *   ldsMaxDegree (device only): largest bank-conflict degree met (Tiled: of the padded tile)
 */
typedef struct cuttStreamCounts {
  double rdInstr, wrInstr, rdInstrIdle, wrInstrIdle;
  double rdLines, wrLines, rdSectors, wrSectors, wrPartialLines, ldsCycles;
  int ldsMaxDegree;
} cuttStreamCounts;

/* CUTT_INVALID_PLAN for an unknown handle, CUTT_INVALID_PARAMETER for a Trivial plan (a copy has
 * no index arithmetic to check) or null pointers.  Synchronises the plan's stream. */
cuttResult cuttCountAddressStream(cuttHandle handle, int numSamples, cuttStreamCounts* onDevice,
                                  cuttStreamCounts* byModel);

/* ---- counters of the cost model (known-answer tests) --------------------- */
int cuttModelGlTransactionsSeg(const int* seg, int n);
int cuttModelGlTransactionsCont(int pos, int n, int accWidth);
void cuttModelCacheLinesSeg(const int* seg, int n, int cacheWidth, int* clFull, int* clPart);
void cuttModelCacheLinesCont(int pos, int n, int cacheWidth, int* clFull, int* clPart);
/* msh: numMsh triples (c, d, ct).  out: sldTran, sstTran, sldReq, sstReq. */
void cuttModelShTransactions(int waveSize, int numBanks, int numThreads, int volMmk, const int* msh,
                             int numMsh, int* out4);

#ifdef __cplusplus
}
#endif

#endif /* CUTT_EXT_H */
