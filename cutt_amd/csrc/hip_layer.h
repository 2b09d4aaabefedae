/*
 * hip_layer.h - the thin C-ABI layer between the host planner and HIP.
 *
 * Everything above this header (cutt_api.cpp, plan.cpp, model.cpp) is plain
 * host C++ that never includes a HIP header; everything that touches the HIP
 * runtime or contains device code lives behind these functions
 * (hip_layer.hip, kernels.hip).  All arguments are plain C types; a stream or
 * event travels as void*.  Every function returns 0 on success or the
 * hipError_t value on failure (cuttHipErrorString turns it into text).
 *
 * It takes the place of three pieces of the reference: the kernel interface
 * src/cuttkernel.h:29-34 (launch configuration + cuttKernel), the device
 * helpers src/CudaUtils.h:44-122 (allocate/copy/memset wrappers) and the
 * event timer src/cuttTimer.h:46-61.
 */
#ifndef CUTT_HIP_LAYER_H
#define CUTT_HIP_LAYER_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Largest tensor rank the kernels accept (the per-rank tables travel as kernel arguments). */
#define CUTT_MAX_RANK 32

/* A launch's workgroups x lanes per workgroup must fit the dispatch packet's 32-bit count of
 * work-items; a larger grid is not refused by the runtime but silently truncated. */
#define CUTT_HIP_MAX_GRID_LANES 0xffffffffull

/* Device facts the planner and the cost model need. */
typedef struct cuttHipDeviceProps {
  int cuCount;              /* compute units */
  int waveSize;             /* lanes per wavefront (64 on gfx950) */
  int maxThreadsPerBlock;
  int maxThreadsPerCU;
  size_t ldsPerBlock;       /* bytes of LDS one workgroup may allocate */
  size_t ldsPerCU;          /* bytes of LDS per compute unit */
  int clockKHz;             /* shader clock */
  int memClockKHz;
  int memBusWidthBits;
  int l2Bytes;
  int maxGridX;
  size_t infinityCacheBytes; /* memory-side cache behind the L2s (256 MB on gfx942/gfx950), 0 if unknown */
  char arch[64];            /* e.g. "gfx950:sramecc+:xnack-" */
} cuttHipDeviceProps;

/*
 * One rank of the "remaining" index set (Mbar): the ranks that neither the
 * input-contiguous set nor the output-contiguous set of a plan covers.  A
 * workgroup's position m in that set is decomposed as
 *   i_k = m % extent_k, m /= extent_k   (ranks in input order)
 * and contributes i_k*strideIn to the input offset and i_k*strideOut to the
 * output offset (offsets in elements).
 */
typedef struct cuttHipMbarDim {
  uint32_t extent;
  uint32_t strideIn;
  uint32_t strideOut;
  /* Division constants, filled by cuttHipFinishMbar: the index along this rank is
   * (m / below) % extent, where `below` is the product of the extents before it; both divisions
   * are multiply-high + shift (see cuttHipDivisor). */
  uint32_t belowMul, extentMul;
  uint32_t ctl; /* belowShift | extentShift << 8 | belowAdd << 16 | extentAdd << 17 */
} cuttHipMbarDim;

typedef struct cuttHipMbar {
  int n;
  cuttHipMbarDim d[CUTT_MAX_RANK];
} cuttHipMbar;

/*
 * Division of a 31-bit number by an invariant divisor d >= 1 without a divide instruction:
 *   n / d == (mulhi32(n, mul) + n * add) >> shift      for every 0 <= n < 2^31.
 * For d >= 2: shift = ceil(log2 d) - 1, mul = ceil(2^(32+shift) / d) (fits 32 bits), add = 0;
 * the rounding error of mul is below d <= 2^(shift+1), so n * error < 2^(32+shift) and the
 * quotient is exact.  d == 1 is mul = 0, add = 1, shift = 0.
 */
typedef struct cuttHipDivisor {
  uint32_t mul;
  uint32_t shift;
  uint32_t add;
} cuttHipDivisor;

cuttHipDivisor cuttHipMakeDivisor(uint32_t d);
/* Host evaluation of the formula above (what the kernels compute). */
uint32_t cuttHipDivide(uint32_t n, cuttHipDivisor dv);
/* Fill the division constants of an Mbar table whose extents are set.  Returns 0, or -1 if the
 * product of the extents does not fit 31 bits. */
int cuttHipFinishMbar(cuttHipMbar* mb);

/*
 * A free numbering of the workgroups of a tiled launch (tile order 7): the logical workgroup index is
 * read as a mixed-radix number, first digit fastest, and every digit belongs to one of the three
 * coordinates of a workgroup - tile along Mm (which = 0), tile along Mk (1), Mbar position (2).  A
 * coordinate is the sum of its digits times their weights; sorted by weight, a coordinate's digits
 * must form a mixed-radix number (weights 1, r0, r0 r1, ...), in whatever order they appear in the
 * index.  The product of a coordinate's radices must reach its extent; indices whose coordinates fall
 * beyond an extent are padding workgroups.  Orders 0-5 are special cases (patches of 2 x 8 tiles walked for 192 Mbar
 * positions in turn: m2 k8 b192 m8 k2 for 16 x 16 tiles).
 */
#define CUTT_MAX_TILE_DIGITS 16
typedef struct cuttHipTileDigit {
  uint32_t radix;
  uint32_t which;       /* 0 tile along Mm, 1 tile along Mk, 2 Mbar position */
  uint32_t weight;      /* the digit's value counts weight times in its coordinate */
  cuttHipDivisor div;   /* division by radix (cuttHipMakeDivisor) */
} cuttHipTileDigit;

/* One digit as the kernels decode it: lane i of a wavefront takes digit i, computes its value
 * (index / below) % radix with two multiply-high divisions (constants as in cuttHipMbarDim) and
 * contributes value * step to the tile coordinates and to the two offsets of the Mbar position. */
typedef struct cuttHipDigitLane {
  uint32_t belowMul, radixMul, ctl, radix;
  uint32_t stepM, stepK;          /* tiles along Mm / Mk per unit of the digit (its weight, or 0) */
  uint32_t strideIn, strideOut;   /* elements per unit of an Mbar digit on the two sides (or 0) */
} cuttHipDigitLane;

typedef struct cuttHipTileDigits {
  int n;
  cuttHipTileDigit d[CUTT_MAX_TILE_DIGITS];
  /* Filled by cuttHipFinishTileDigits from d[] and the plan's Mbar table.  lanes = 1 if every Mbar
   * digit stays inside one Mbar rank, so that the offsets are linear in the digits: the kernels then
   * decode a workgroup index with lane[] in one step; otherwise (lanes = 0) digit by digit. */
  int lanes;
  uint32_t total;                 /* product of the radices: indices from here on are padding */
  cuttHipDigitLane lane[CUTT_MAX_TILE_DIGITS];
} cuttHipTileDigits;
/* Derive lanes, total and lane[] of a digit list from d[] and the Mbar table of the same plan
 * (returns 0; a list that cannot be decoded in one step gets lanes = 0). */
int cuttHipFinishTileDigits(cuttHipTileDigits* dg, const cuttHipMbar* mb);

/*
 * Offsets of the rows of a tile when a tile axis runs over several fused ranks: row index i along the
 * set (first rank fastest) has the offset sum_k ((i / prod_{j<k} extent_j) % extent_k) * stride_k.
 * n = 0: the axis is a single rank and the offset is i * stride (strideInK / strideOutM of the
 * arguments).
 */
#define CUTT_MAX_TILE_SET 4
typedef struct cuttHipRowRadix {
  int n;
  uint32_t extent[CUTT_MAX_TILE_SET];
  uint32_t stride[CUTT_MAX_TILE_SET];
  cuttHipDivisor div[CUTT_MAX_TILE_SET]; /* division by extent[k] */
} cuttHipRowRadix;

/*
 * Tiled method: a batch of 2-D transposes between the ranks that lead the input (Mm: fused extent
 * volMm, contiguous in the input) and the ranks that lead the output (Mk: fused extent volMk,
 * contiguous in the output), staged through a padded 64x64 LDS tile.  One workgroup per (tile, Mbar
 * position).  With one rank on each side (rowsK.n == rowsM.n == 0) row k of a tile lies
 * k * strideInK into the input and row m lies m * strideOutM into the output; with several ranks on a
 * side the rows' offsets follow rowsK / rowsM.
 */
typedef struct cuttHipTiledArgs {
  int elemSize;       /* 4 or 8 */
  int volMm, volMk;
  uint32_t strideInK;
  uint32_t strideOutM;
  int tilesM, tilesK; /* ceil(volMm/64), ceil(volMk/64) */
  int volMbar;
  int order;          /* logical numbering of the workgroups: 0 = Mbar fastest, 1 = tiles along Mm
                         fastest, 2 = tiles along Mk fastest, 3 / 4 = superM x superK super-tiles with the
                         tiles along Mm / along Mk running fastest inside and between them; 5 = as 3,
                         but every super-tile is visited for all Mbar positions in turn; 6 = as 5 with
                         the super-tiles numbered along Mk first and each row of them rotated by its
                         index along Mm (the XCDs then work on different columns at one time); 7 = the
                         mixed-radix numbering in `digits` */
  uint32_t xcdChunk;  /* 0: workgroup b is logical position b; else (b % 8)*xcdChunk + b/8, and the
                         grid has 8*xcdChunk workgroups */
  uint32_t superM, superK;
  int cachePolicy;    /* 0 = default, 1 = non-temporal loads, 3 = non-temporal loads and stores */
  int grouped;        /* 0: a lane has all 16 rows of its tile in flight at once; 1: four at a time
                         (each group of 16 tile rows is waited for before the next is requested) */
  int alignedStores;  /* 1: every tile row stores its own 64-element window of the output run, shifted
                         so that it starts on a 128-byte line; tilesK is then
                         ceil((volMk + 128/elemSize - 1) / 64) and grouped must be 0 */
  cuttHipRowRadix rowsK; /* Mk index -> input offset (n == 0: index * strideInK) */
  cuttHipRowRadix rowsM; /* Mm index -> output offset (n == 0: index * strideOutM) */
  cuttHipTileDigits digits; /* order 7 only */
  cuttHipMbar mbar;
} cuttHipTiledArgs;

/*
 * TiledCopy method: rank 0 keeps its place, so rows along rank 0 (extent
 * volMm) are copied; the second output rank (extent volMk, input stride
 * strideInK, output stride strideOutK) is the other tile axis.  No LDS.
 */
typedef struct cuttHipTiledCopyArgs {
  int elemSize;
  int volMm, volMk;
  uint32_t strideInK;
  uint32_t strideOutK;
  int tilesM, tilesK;
  int volMbar;
  int order;
  uint32_t xcdChunk;
  uint32_t superM, superK;
  int cachePolicy;
  cuttHipTileDigits digits; /* order 7 only */
  cuttHipMbar mbar;
} cuttHipTiledCopyArgs;

/*
 * Index-remap tables of a Packed / PackedSplit plan for one slab-size class (device pointers).
 * The staged block holds `vol` elements.  In input-compact order the block is vol/inCont
 * contiguous runs of inCont elements: element p is read from input offset
 * rowIn[p / inCont] + p % inCont and parked in LDS slot p + (p >> padShift).  In output-compact
 * order it is vol/outCont runs of outCont elements: element q is written to output offset
 * rowOut[q / outCont] + q % outCont and taken from LDS slot shIdx[q] (padding included).
 * A workgroup derives its lanes' offsets once and keeps them in registers for all the work
 * items it handles; one offset per run instead of one per element keeps the tables small
 * (2 bytes per element plus 4 per run), since every workgroup reads them through the L2.
 */
typedef struct cuttHipPackedClass {
  int vol;
  int inCont, outCont;       /* contiguous run lengths; both divide vol */
  cuttHipDivisor inDiv, outDiv; /* divisions by inCont / outCont (cuttHipMakeDivisor) */
  const uint32_t* rowIn;     /* vol / inCont entries */
  const uint32_t* rowOut;    /* vol / outCont entries */
  const uint16_t* shIdx;     /* vol entries */
} cuttHipPackedClass;

/* One split rank of a PackedSplit plan: the rank is cut into numSplit slabs; slab s covers
 * [s*slabFloor + min(s, slabRem), ...) and has slabFloor + (s < slabRem) entries.  An unused
 * slot has numSplit 1, slabRem 0 and zero strides. */
typedef struct cuttHipSplitRank {
  int numSplit;
  int slabFloor, slabRem;
  uint32_t strideIn, strideOut; /* global strides of the rank */
  cuttHipDivisor div;           /* division by numSplit (cuttHipMakeDivisor) */
} cuttHipSplitRank;

/*
 * Packed and PackedSplit methods.  A staged block is the index set Mmk with up to two of its
 * ranks cut into slabs (typically the last rank of the input-contiguous set and the last rank of
 * the output-contiguous set, which makes the block a 2-D tile over fused rank sets).  Work items
 * are (Mbar position m, slab s1, slab s0); workgroup b handles the items numbered
 * [b*itemsPerBlock, (b+1)*itemsPerBlock).  Two numberings (itemOrder):
 *   0: w = (m*numSplit1 + s1)*numSplit0 + s0 - a workgroup walks neighbouring slabs;
 *   1: w = ((mb*numSplit1 + s1)*numSplit0 + s0)*itemsPerBlock + mi with m = mb*itemsPerBlock + mi
 *      (numbers whose m >= volMbar are skipped) - a workgroup keeps its slabs and walks
 *      itemsPerBlock Mbar positions, neighbouring workgroups have neighbouring slabs.
 *   2: numbered as in 0, handed out differently: the workgroups of one XCD (of the whole grid when
 *      xcdChunk is 0) take the numbers of their chunk in turn - the workgroup with index q inside
 *      a chunk of B workgroups handles chunkStart + q, chunkStart + q + B, ... - so that the items
 *      in flight at one time are neighbours in memory and a workgroup's next item lies one round
 *      ahead.
 * The slab sizes select the table class: cls[(s0 < slabRem0) + 2*(s1 < slabRem1)]; a workgroup that
 * meets another class reloads its lanes' table entries (a round trip to memory), which order 1
 * never does (and order 2 does most often, when slabs of different sizes exist).  Packed is the case without split ranks.
 */
typedef struct cuttHipPackedArgs {
  int elemSize;
  int numThreads;
  int volMbar;
  cuttHipSplitRank split[2];
  int itemsPerBlock;
  int itemOrder;       /* numbering of the work items, see above */
  int elemsPerThread;  /* 1, 2, 4, 8 or (4-byte elements only) 16: numThreads*elemsPerThread >= vol of every class */
  int padShift;        /* LDS slot(p) = p + (p >> padShift); 31 = no padding */
  int ldsElems;        /* element slots in the LDS data buffer (padding included) */
  int maxVol;          /* largest class volume */
  uint32_t xcdChunk;   /* 0: workgroup b is logical block b; else logical block = (b % 8)*xcdChunk + b/8
                          and the grid has 8*xcdChunk workgroups */
  int cachePolicy;     /* 0 = default, 1 = non-temporal loads, 3 = non-temporal loads and stores */
  long long volume;    /* elements from the first to the last one of the tensor, on its wider side (bounds every offset) */
  int wideOffsets;     /* 0: the tensor is below 4 GB and the kernel keeps 32-bit byte offsets;
                          1: element offsets with 64-bit address arithmetic (required from 4 GB on) */
  cuttHipPackedClass cls[4];
  cuttHipMbar mbar;
} cuttHipPackedArgs;

/* Work-item numbers of these arguments (some of them empty in order 1), or -1 if beyond 31 bits. */
long long cuttHipPackedItemNumbers(const cuttHipPackedArgs* args);
/* Work-item number w -> Mbar position, slab indices and table class, as the kernel computes them;
 * returns 0 if the number is empty (order 1, m beyond volMbar). */
int cuttHipDecodeItem(const cuttHipPackedArgs* args, uint32_t w, uint32_t* m, uint32_t* s0, uint32_t* s1, int* cls);
/* Bytes of LDS the packed kernel needs for these arguments. */
size_t cuttHipPackedLdsBytes(const cuttHipPackedArgs* a);
/* Vector registers per lane of the packed kernel instance for this element size, elements per lane
 * and offset width, as built (a table kept beside the kernel; needs no GPU).  The planner derives
 * the resident wavefronts per CU from it: min(8, 512 / roundup8(registers)) per SIMD, 4 SIMDs. */
int cuttHipPackedRegsPerLane(int elemSize, int elemsPerThread, int wideOffsets);
/* The same number asked of the HIP runtime for the loaded code object (needs a GPU); -1 on error. */
int cuttHipPackedRegsPerLaneLoaded(int elemSize, int elemsPerThread, int wideOffsets);

/* ---- device, memory, stream and event helpers ---------------------------- */
int cuttHipGetDevice(int* device);
int cuttHipGetDeviceProps(int device, cuttHipDeviceProps* props);
int cuttHipMalloc(void** ptr, size_t bytes);
int cuttHipFree(void* ptr);
/* How often this process has called cuttHipMalloc and cuttHipMemcpyHtoD so far (tests read them
 * before and after a call that must neither allocate nor upload). */
void cuttHipCallCounts(unsigned long long* mallocs, unsigned long long* uploads);
/* Host to device copy that has completed when the call returns. */
int cuttHipMemcpyHtoD(void* dst, const void* src, size_t bytes);
int cuttHipMemcpyDtoDAsync(void* dst, const void* src, size_t bytes, void* stream);
int cuttHipMemsetAsync(void* dst, int value, size_t bytes, void* stream);
int cuttHipDeviceSynchronize(void);
int cuttHipEventCreate(void** event);
int cuttHipEventDestroy(void* event);
int cuttHipEventRecord(void* event, void* stream);
int cuttHipEventSynchronize(void* event);
int cuttHipEventElapsedMs(void* start, void* stop, float* ms);
const char* cuttHipErrorString(int err);

/* ---- kernel launches (asynchronous on `stream`) --------------------------
 * A plan's arguments are checked once, when the plan is activated (cuttHipValidate*: shapes, grid,
 * division constants, table pointers; 0 or a hipError_t value); the launch functions then only
 * compute the grid and launch, and return the launch call's own result.  Launching arguments that
 * did not pass their check is undefined. */
int cuttHipValidateTiled(const cuttHipTiledArgs* args);
int cuttHipValidateTiledCopy(const cuttHipTiledCopyArgs* args);
int cuttHipValidatePacked(const cuttHipPackedArgs* args);
/* Workgroups of a tiled launch with these arguments (padding workgroups included), 0 if they have no valid grid. */
long long cuttHipTiledGrid(const cuttHipTiledArgs* args);
long long cuttHipTiledCopyGrid(const cuttHipTiledCopyArgs* args);
int cuttHipLaunchTiled(const cuttHipTiledArgs* args, const void* in, void* out, void* stream);
int cuttHipLaunchTiledCopy(const cuttHipTiledCopyArgs* args, const void* in, void* out, void* stream);
int cuttHipLaunchPacked(const cuttHipPackedArgs* args, const void* in, void* out, void* stream);
/*
 * Index tables of one slab class built on the device (for callers that may not allocate or copy):
 * entry i of table l is the mixed-radix sum over list[l] (first entry fastest) of index * stride;
 * l = 0 fills rowIn (count[0] entries), l = 1 rowOut (count[1]), l = 2 the LDS gather slots
 * (count[2] entries, stored as position + (position >> padShift)).
 */
typedef struct cuttHipRadixList {
  int n;
  uint32_t extent[CUTT_MAX_RANK];
  uint32_t stride[CUTT_MAX_RANK];
} cuttHipRadixList;

typedef struct cuttHipTableBuildArgs {
  uint32_t count[3];
  int padShift;
  cuttHipRadixList list[3];
  uint32_t* rowIn;
  uint32_t* rowOut;
  uint16_t* shIdx;
} cuttHipTableBuildArgs;

int cuttHipLaunchTableBuild(const cuttHipTableBuildArgs* args, void* stream);

/*
 * The library's static scratch memory on the current device (a __device__ array in the code
 * object, CUTT_HIP_SCRATCH_BYTES bytes, 256-byte aligned): its device address, looked up once per
 * device.  Every caller on one device shares the same array.  0 or a hipError_t value.
 */
#define CUTT_HIP_SCRATCH_BYTES (1u << 20)
int cuttHipScratch(void** ptr, size_t* bytes);

/*
 * What the address stream of a plan's kernel amounts to, counted on the device by kernels that
 * replay it (count_kernels.hip): wavefront-level load and store instructions that carry data, those
 * whose lanes all repeat an edge element ("idle"), distinct 128-byte lines and 32-byte sectors per
 * instruction summed over the launch, partly written lines at the ends of the output runs, LDS
 * cycles of the packed kernel's gathers, and the largest LDS bank-conflict degree met.
 */
typedef struct cuttHipStreamCounts {
  unsigned long long rdInstr, wrInstr, rdInstrIdle, wrInstrIdle;
  unsigned long long rdLines, wrLines, rdSectors, wrSectors, wrPartialLines, ldsCycles;
  unsigned int ldsMaxDegree;
} cuttHipStreamCounts;

/* Launch the counting kernel for these (validated) arguments on `stream`, wait, return the totals. */
int cuttHipCountTiled(const cuttHipTiledArgs* args, cuttHipStreamCounts* out, void* stream);
int cuttHipCountTiledCopy(const cuttHipTiledCopyArgs* args, cuttHipStreamCounts* out, void* stream);
int cuttHipCountPacked(const cuttHipPackedArgs* args, cuttHipStreamCounts* out, void* stream);

/* Plain copy of `bytes` bytes (a multiple of 4) for the Trivial method; cachePolicy as above. */
int cuttHipLaunchCopy(const void* in, void* out, size_t bytes, int cachePolicy, void* stream);
/* One-time kernel attribute setup of the packed kernels on the current device (idempotent). */
int cuttHipPreparePacked(void);

#ifdef __cplusplus
}
#endif

#endif /* CUTT_HIP_LAYER_H */
