/*
 * kernels.hip - transpose kernels for gfx950 (64-lane wavefronts) and their
 * launch functions.
 *
 * Four data paths, matching the reference's method set
 * (reference src/cuttkernel.cu:38-118 Tiled, :123-222 Packed, :230-347
 * PackedSplit, :356-426 TiledCopy), written for CDNA4 rather than translated:
 *
 *  - every kernel moves opaque 4- or 8-byte words (uint32_t / uint64_t), one
 *    word per lane per access, so a wavefront touches 256 or 512 contiguous
 *    bytes per instruction when the run is long enough;
 *  - the per-rank decomposition of a workgroup's Mbar position is wave-uniform:
 *    lane k owns rank k, divides by precomputed multiply-high constants and the
 *    wavefront sums the contributions with DPP adds (mbar_decode.h);
 *  - Tiled stages a 64x64 tile in LDS padded to 65 columns (conflict-free for
 *    both 4- and 8-byte words); each lane keeps 16 loads in flight; edges are handled by
 *    clamping indices, not by branches, so the memory instructions stay back to back;
 *  - Packed/PackedSplit take their index remap from tables the planner precomputed in device
 *    memory (one input offset per contiguous input run, one output offset per contiguous output
 *    run, an LDS gather slot per staged element); a workgroup derives its lanes' offsets once and
 *    keeps them in registers while it loops over its work items, so the loop body is load, LDS
 *    write, LDS read, store; the LDS buffer is skewed by one slot per 2^padShift to break
 *    power-of-two bank strides;
 *  - workgroups are short-lived and small (a tile, or a few Mbar positions),
 *    thousands are in flight: on this chip that streams faster than a
 *    persistent grid-stride loop.
 *
 * All offsets are unsigned 32-bit element offsets from the pointers of the launch (one launch
 * spans fewer than 2^32 elements on either side - a larger tensor comes in pieces -; every true
 * offset is below that span, so the modular sums are exact); the packed kernel turns them into
 * 32-bit byte offsets from a wave-uniform base when the span is below 4 GB.
 */
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <tuple>
#include <type_traits>

#include "hip_layer.h"
#include "mbar_decode.h"
#include "packed_items.h"
#include "tile_order.h"

using namespace cutt;

namespace {

// Cache policy of the global accesses, a kernel template parameter NT: bit 0 = non-temporal
// (streaming) loads, bit 1 = non-temporal stores.  The input is read once, so streaming loads keep
// the L2 free for the output lines that neighbouring workgroups still have to complete; streaming
// stores pay off only when every written run covers whole 128-byte lines.
template <int NT, typename T>
__device__ __forceinline__ T ldg(const T* p) {
  if constexpr (NT & 1) return __builtin_nontemporal_load(p);
  else return *p;
}
template <int NT, typename T>
__device__ __forceinline__ void stg(T* p, T v) {
  if constexpr (NT & 2) __builtin_nontemporal_store(v, p);
  else *p = v;
}

// Blocks the wave until its outstanding global loads have returned and its stores have been
// acknowledged (the vector memory counter reaches zero); also a barrier for the compiler.
__device__ __forceinline__ void waitForGlobalAccesses() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---------------------------------------------------------------------------
// Tiled: 64x64 tile through padded LDS.
// ---------------------------------------------------------------------------
// GROUPED: the four row groups of a lane go one after the other - request 4 rows, wait, stage them,
// request the next 4; store 4 rows, wait, store the next 4 - instead of all 16 rows at once.  That
// quarters what a workgroup has in flight.  When tile rows start off the 128-byte grid (4-byte
// elements, large tensors) it is 3-11 % faster: the neighbouring tiles' requests for a shared line
// then arrive while the line is still in the L2.  On aligned or cache-resident tensors it is up to
// 10 % slower, so the planner decides (cuttHipTiledArgs.grouped).
//
// FUSED: a tile axis runs over several fused ranks (the ranks that lead the input on the Mm side, the
// ranks that lead the output on the Mk side), so the rows of a tile are not equally far apart.  Lane l
// derives the offset of row l of either axis with a short mixed-radix decode (tileRowOffsets) and the
// wave picks a row's offset out of that lane; the elements of a row are contiguous as before.
template <typename T, int NT, bool GROUPED, bool FUSED>
__global__ __launch_bounds__(kTileThreads) void tiledKernel(const cuttHipTiledArgs a,
                                                            const T* __restrict__ in,
                                                            T* __restrict__ out) {
  __shared__ T tile[kTile][kTile + 1];

  uint32_t tm, tk, offIn, offOut;
  if (!locateTile(a, tm, tk, offIn, offOut)) return;

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  // tile geometry, clamped edges, skipped row groups: tile_order.h
  const TileLanes t = tileLanes<FUSED>(a, tm, tk, offIn, offOut, lane, wave);

  // Read: lanes run along the input-contiguous axis (Mm), rows along Mk.
  {
    T v[kTileRows];
#pragma unroll
    for (int g = 0; g < kRowGroups; g++) {
      if ((uint32_t)g < t.groupsK) {
#pragma unroll
        for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) v[j] = ldg<NT>(in + tileReadElem<FUSED>(t, a, wave, j));
        if constexpr (GROUPED) {
          waitForGlobalAccesses();
#pragma unroll
          for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) {
            const uint32_t r = min(wave + kWaves * j, t.wK);
            tile[r][t.cx] = v[j];
          }
        }
      }
    }
    if constexpr (!GROUPED) {
#pragma unroll
      for (int g = 0; g < kRowGroups; g++) {
        if ((uint32_t)g < t.groupsK) {
#pragma unroll
          for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) {
            const uint32_t r = min(wave + kWaves * j, t.wK);
            tile[r][t.cx] = v[j];
          }
        }
      }
    }
  }
  __syncthreads();
  // Write: lanes run along the output-contiguous axis (Mk), rows along Mm.
  {
    T v[kTileRows];
#pragma unroll
    for (int g = 0; g < kRowGroups; g++) {
      if ((uint32_t)g < t.groupsM) {
#pragma unroll
        for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) {
          const uint32_t r = min(wave + kWaves * j, t.wM);
          v[j] = tile[t.ck][r];
        }
        if constexpr (GROUPED) {
#pragma unroll
          for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) stg<NT>(out + tileWriteElem<FUSED>(t, a, wave, j), v[j]);
          waitForGlobalAccesses();
        }
      }
    }
    if constexpr (!GROUPED) {
#pragma unroll
      for (int g = 0; g < kRowGroups; g++) {
        if ((uint32_t)g < t.groupsM) {
#pragma unroll
          for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) stg<NT>(out + tileWriteElem<FUSED>(t, a, wave, j), v[j]);
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Tiled with line-aligned stores.  When the output rows (runs along Mk) start off the 128-byte
// grid, the 64-wide store of a tile row covers three lines, two of them partly, and the tile next
// door along Mk completes them later.  Here every row of a tile takes its own window of 64
// elements along Mk: row m, whose output run starts s_m elements past a line boundary, stores the
// elements [64 tk - s_m, 64 tk - s_m + 64) of its run, so every store of a wave is two whole lines
// (except at the two ends of a run).  The windows of the rows of a tile differ by up to one line,
// so the workgroup reads up to 64 + (elements per line - 1) rows along Mk into a taller LDS tile;
// the rows in the fringe are also read by the tile next door (from the L2).  The grid has
// ceil((volMk + elements per line - 1) / 64) tiles along Mk.
template <typename T>
constexpr int kLineElems = 128 / (int)sizeof(T);
template <typename T>
constexpr int kAlignedRows = kTile + kLineElems<T> - 1;  // rows along Mk that a workgroup may need

template <typename T, int NT>
__global__ __launch_bounds__(kTileThreads) void tiledAlignedKernel(const cuttHipTiledArgs a,
                                                                   const T* __restrict__ in,
                                                                   T* __restrict__ out) {
  constexpr int LE = kLineElems<T>;
  constexpr int ROWS = kAlignedRows<T>;
  constexpr int RD = (ROWS + kWaves - 1) / kWaves;  // rows a wave reads at most
  __shared__ T tile[ROWS][kTile + 1];

  uint32_t tm, tk, offIn, offOut;
  if (!locateTile(a, tm, tk, offIn, offOut)) return;

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t m0 = tm * kTile;
  const int32_t kBase = (int32_t)(tk * kTile) - (LE - 1);  // first row along Mk the tile may need
  const uint32_t volMm = a.volMm, volMk = a.volMk;
  const uint32_t wM = min((uint32_t)kTile, volMm - m0) - 1;
  const uint32_t groupsM = (wM >> 4) + 1;

  // Misalignment of output row m in elements (the low bits of its element address).  Over the
  // rows of a tile it takes the values c + j g (mod LE), g = gcd(strideOutM, LE): the rows along
  // Mk that some row of the tile needs are kBase + [LE - 1 - sMax, LE - 1 - sMin + 64).
  const uint32_t outWord = (uint32_t)(reinterpret_cast<uintptr_t>(out) / sizeof(T)) + offOut;
  const uint32_t g = min((uint32_t)LE, a.strideOutM & (0u - a.strideOutM));  // lowest set bit, capped
  const uint32_t sMin = (outWord + m0 * a.strideOutM) & (g - 1);
  const uint32_t sMax = sMin + (LE - g);
  const uint32_t rowLo = (LE - 1) - sMax, rowHi = (LE - 1) - sMin + kTile;  // [rowLo, rowHi)

  // Read: lanes run along input rank 0, rows along Mk (clamped to the rank's ends).
  {
    const uint32_t cx = min(lane, wM);
    const T* src = in + (offIn + m0 + cx);
    T v[RD];
#pragma unroll
    for (int j = 0; j < RD; j++) {
      const uint32_t row = wave + kWaves * j;
      if (row >= rowLo && row < rowHi) {  // uniform over the wave
        const int32_t k = min(max(kBase + (int32_t)row, 0), (int32_t)volMk - 1);
        v[j] = ldg<NT>(src + (uint32_t)k * a.strideInK);
      }
    }
#pragma unroll
    for (int j = 0; j < RD; j++) {
      const uint32_t row = wave + kWaves * j;
      if (row >= rowLo && row < rowHi) tile[row][cx] = v[j];
    }
  }
  __syncthreads();
  // Write: lanes run along Mk inside the row's own window.
  {
    T v[kTileRows];
    uint32_t dstOff[kTileRows];
#pragma unroll
    for (int gI = 0; gI < kRowGroups; gI++) {
      if ((uint32_t)gI < groupsM) {
#pragma unroll
        for (int j = gI * kGroupRows; j < (gI + 1) * kGroupRows; j++) {
          const uint32_t r = min(wave + kWaves * j, wM);
          const uint32_t rowStart = offOut + (m0 + r) * a.strideOutM;
          const uint32_t sRow = (outWord - offOut + rowStart) & (LE - 1);
          const int32_t k = min(max((int32_t)(tk * kTile) - (int32_t)sRow + (int32_t)lane, 0), (int32_t)volMk - 1);
          // (a window that lies wholly beyond the run's end repeats the run's last element, which
          // every LDS row from rowLo on holds in that case)
          v[j] = tile[max(k - kBase, (int32_t)rowLo)][r];
          dstOff[j] = rowStart + (uint32_t)k;
        }
      }
    }
#pragma unroll
    for (int gI = 0; gI < kRowGroups; gI++) {
      if ((uint32_t)gI < groupsM) {
#pragma unroll
        for (int j = gI * kGroupRows; j < (gI + 1) * kGroupRows; j++) stg<NT>(out + dstOff[j], v[j]);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// TiledCopy: rank 0 stays in front; rows are copied through registers.
// ---------------------------------------------------------------------------
template <typename T, int NT>
__global__ __launch_bounds__(kTileThreads) void tiledCopyKernel(const cuttHipTiledCopyArgs a,
                                                                const T* __restrict__ in,
                                                                T* __restrict__ out) {
  uint32_t tm, tk, offIn, offOut;
  if (!locateTile(a, tm, tk, offIn, offOut)) return;

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t m0 = tm * kTile, k0 = tk * kTile;
  // Clamped indices instead of branches, as in the tiled kernel.
  const uint32_t cx = min(lane, min((uint32_t)kTile, (uint32_t)a.volMm - m0) - 1);
  const uint32_t wK = min((uint32_t)kTile, (uint32_t)a.volMk - k0) - 1;
  const T* src = in + (offIn + m0 + cx);
  T* dst = out + (offOut + m0 + cx);

  // Row groups that lie beyond the tile's valid rows are skipped, as in the tiled kernel.
  const uint32_t groupsK = (wK >> 4) + 1;
  T v[kTileRows];
#pragma unroll
  for (int g = 0; g < kRowGroups; g++) {
    if ((uint32_t)g < groupsK) {
#pragma unroll
      for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) {
        const uint32_t r = min(wave + kWaves * j, wK);
        v[j] = ldg<NT>(src + (k0 + r) * a.strideInK);
      }
    }
  }
#pragma unroll
  for (int g = 0; g < kRowGroups; g++) {
    if ((uint32_t)g < groupsK) {
#pragma unroll
      for (int j = g * kGroupRows; j < (g + 1) * kGroupRows; j++) {
        const uint32_t r = min(wave + kWaves * j, wK);
        stg<NT>(dst + (k0 + r) * a.strideOutK, v[j]);
      }
    }
  }
}

// ---------------------------------------------------------------------------
// Packed / PackedSplit: stage a block of Mmk through LDS with remap tables.
// ---------------------------------------------------------------------------

// E = elements per lane.  Every lane keeps its E table entries in registers, so that the loop
// over work items does no index arithmetic beyond adding the item's base offsets; the loop is
// software-pipelined (an item's loads are in flight while the previous one is gathered and stored).
// WIDE = false: the tensor is smaller than 4 GB, so the lanes keep 32-bit byte offsets and every
// access is "uniform 64-bit base + 32-bit lane offset" (no per-access 64-bit address registers).  WIDE = true:
// element offsets and 64-bit address arithmetic.
// (The 8-byte instance with 8 elements per lane sits at the edge of a register granule: it is held to the 80
// registers that let six of its waves share a SIMD; the other instances get what the compiler gives them.)
template <typename T, int E, bool WIDE>
constexpr int kPackedMinWaves = (sizeof(T) == 8 && E == 8 && !WIDE) ? 6 : 1;

template <typename T, int E, int NT, bool WIDE>
__global__ __launch_bounds__(1024, (kPackedMinWaves<T, E, WIDE>)) void packedKernel(const cuttHipPackedArgs a, const T* __restrict__ in,
                             T* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char ldsRaw[];
  constexpr uint32_t kScale = WIDE ? 1u : (uint32_t)sizeof(T);

  const uint32_t tid = threadIdx.x;
  const uint32_t nt = blockDim.x;
  // which work items this workgroup handles, and where an item lies: packed_items.h
  const PackedItems items = packedItems(a);
  const uint32_t count = items.count;
  const int padShift = a.padShift;

  // Lanes whose element index lies beyond the block repeat the block's last element (same
  // addresses, same value), so that the code below has no branches and every lane's E loads go
  // out back to back.
  uint32_t inOff[E], outOff[E];  // global offsets: bytes (narrow) or elements (wide)
  uint32_t shSlot[E];            // byte offset of the LDS slot an output element is taken from
  uint32_t last = 0;             // last element index of the class whose data is being loaded
  const MbarLane mbarLane = loadMbarLane(a.mbar, tid & 63);

  auto locate = [&](uint32_t i, int& c, uint32_t& offIn, uint32_t& offOut) __attribute__((always_inline)) {
    packedLocate(a, items, mbarLane, i, c, offIn, offOut);
  };
  // The lane's table entries of class c: the read side (input offsets, element count) and the
  // write side (output offsets, LDS gather slots) are fetched separately, because the next item's
  // loads go out while the current item's stores are still to come.
  auto loadReadSide = [&](int c) __attribute__((always_inline)) {
    const cuttHipPackedClass& k = a.cls[c];
    last = (uint32_t)k.vol - 1;
#pragma unroll
    for (int j = 0; j < E; j++) inOff[j] = packedInElem(k, min(tid + j * nt, last)) * kScale;
  };
  auto loadWriteSide = [&](int c) __attribute__((always_inline)) {
    const cuttHipPackedClass& k = a.cls[c];
    const uint32_t lastP = (uint32_t)k.vol - 1;
    const uint16_t* gSh = k.shIdx;
#pragma unroll
    for (int j = 0; j < E; j++) {
      const uint32_t p = min(tid + j * nt, lastP);
      const uint32_t sh = *reinterpret_cast<const uint16_t*>(reinterpret_cast<const unsigned char*>(gSh) + p * 2u);
      outOff[j] = packedOutElem(k, p) * kScale;
      shSlot[j] = sh * (uint32_t)sizeof(T);
    }
  };
  T v[E];  // data on its way in: global memory -> registers -> LDS
  auto issueLoads = [&](uint32_t offIn) __attribute__((always_inline)) {
    const unsigned char* srcB = reinterpret_cast<const unsigned char*>(in + offIn);  // wave-uniform base
#pragma unroll
    for (int j = 0; j < E; j++) {
      if (WIDE)
        v[j] = ldg<NT>(reinterpret_cast<const T*>(srcB) + inOff[j]);
      else
        v[j] = ldg<NT>(reinterpret_cast<const T*>(srcB + inOff[j]));
    }
  };
  // The slot of element p is p + (p >> padShift).  It is recomputed for every item from a value
  // the compiler cannot see through, so that it does not park E more registers.
  auto stage = [&]() __attribute__((always_inline)) {
    uint32_t tv = tid;
    asm volatile("" : "+v"(tv));
#pragma unroll
    for (int j = 0; j < E; j++) {
      const uint32_t p = min(tv + j * nt, last);
      *reinterpret_cast<T*>(ldsRaw + (p + (p >> padShift)) * (uint32_t)sizeof(T)) = v[j];
    }
  };
  auto gatherAndStore = [&](uint32_t offOut) __attribute__((always_inline)) {
    unsigned char* dstB = reinterpret_cast<unsigned char*>(out + offOut);
    T u[E];
#pragma unroll
    for (int j = 0; j < E; j++) u[j] = *reinterpret_cast<const T*>(ldsRaw + shSlot[j]);
#pragma unroll
    for (int j = 0; j < E; j++) {
      if (WIDE)
        stg<NT>(reinterpret_cast<T*>(dstB) + outOff[j], u[j]);
      else
        stg<NT>(reinterpret_cast<T*>(dstB + outOff[j]), u[j]);
    }
  };

  // Software pipeline over the workgroup's items: the loads of item w+1 are issued before the LDS
  // gather and the stores of item w, so they overlap, and the wait for them (the memory counter
  // counts loads and stores in issue order) does not also wait for those stores to complete.
  if (count == 0) return;
  uint32_t w = 0, offIn, offOut;  // index of the item among the workgroup's own
  int cls;
  locate(w, cls, offIn, offOut);
  loadReadSide(cls);
  issueLoads(offIn);
  loadWriteSide(cls);  // after the data loads are out: its latency hides behind theirs
  stage();
  for (;;) {
    if (w + 1 >= count) {  // last item: nothing to fetch ahead
      __syncthreads();
      gatherAndStore(offOut);
      break;
    }
    int clsNext;
    uint32_t offInNext, offOutNext;
    locate(w + 1, clsNext, offInNext, offOutNext);
    // the slab class changes at most a few times per workgroup (wave-uniform tests)
    if (clsNext != cls) loadReadSide(clsNext);
    issueLoads(offInNext);
    __syncthreads();  // item w is complete in the LDS buffer
    gatherAndStore(offOut);
    if (clsNext != cls) {
      loadWriteSide(clsNext);
      cls = clsNext;
    }
    __syncthreads();  // every lane has taken its elements of item w out of the buffer
    stage();
    w++;
    offOut = offOutNext;
  }
}

// The table must carry the division constants cuttHipFinishMbar derives from its extents.
bool mbarOk(const cuttHipMbar& mb) {
  cuttHipMbar want = mb;
  if (cuttHipFinishMbar(&want) != 0) return false;
  for (int k = 0; k < CUTT_MAX_RANK; k++)
    if (want.d[k].belowMul != mb.d[k].belowMul || want.d[k].extentMul != mb.d[k].extentMul ||
        want.d[k].ctl != mb.d[k].ctl)
      return false;
  return true;
}

bool divisorOk(const cuttHipDivisor& dv, uint32_t d) {
  const cuttHipDivisor want = cuttHipMakeDivisor(d);
  return dv.mul == want.mul && dv.shift == want.shift && dv.add == want.add;
}

// Number of workgroups of a tiled launch; checks the ordering parameters.
bool tileGrid(int order, int tilesM, int tilesK, int volMbar, uint32_t xcdChunk, uint32_t superM,
              uint32_t superK, const cuttHipTileDigits& dg, const cuttHipMbar& mbar, uint64_t& blocks) {
  uint64_t logical = (uint64_t)tilesM * tilesK * (uint64_t)volMbar;
  if (order == 7) {
    if (dg.n < 1 || dg.n > CUTT_MAX_TILE_DIGITS) return false;
    logical = 1;
    for (int i = 0; i < dg.n; i++) {
      const cuttHipTileDigit& d = dg.d[i];
      if (d.radix < 1 || d.which > 2 || !divisorOk(d.div, d.radix)) return false;
      logical *= d.radix;
      if (logical > 0x7fffffffull) return false;  // the decode divides 31-bit numbers
    }
    // per coordinate the digits, taken by growing weight, must be a mixed-radix number that reaches the extent
    const uint64_t extent[3] = {(uint64_t)tilesM, (uint64_t)tilesK, (uint64_t)volMbar};
    for (uint32_t w = 0; w < 3; w++) {
      uint64_t span = 1;
      for (;;) {
        int next = -1;
        for (int i = 0; i < dg.n; i++)
          if (dg.d[i].which == w && dg.d[i].weight == span && dg.d[i].radix > 1 && (next < 0 || dg.d[i].radix > dg.d[next].radix)) next = i;
        if (next < 0) break;
        span *= dg.d[next].radix;
      }
      uint64_t all = 1;
      for (int i = 0; i < dg.n; i++)
        if (dg.d[i].which == w && dg.d[i].radix > 1) all *= dg.d[i].radix;
      if (span != all || span < extent[w]) return false;
    }
    // what the kernels decode with must be what cuttHipFinishTileDigits derives from the list
    // (a list without lanes is decoded digit by digit, which needs none of this)
    if (dg.lanes) {
      cuttHipTileDigits want = dg;
      if (cuttHipFinishTileDigits(&want, &mbar) != 0 || want.lanes != 1 || want.total != dg.total ||
          std::memcmp(want.lane, dg.lane, sizeof(dg.lane)) != 0)
        return false;
    }
  } else if (order >= 3) {
    if (superM < 1 || superK < 1) return false;
    logical = (uint64_t)((tilesM + superM - 1) / superM) * ((tilesK + superK - 1) / superK) * superM * superK *
              (uint64_t)volMbar;
  }
  blocks = logical;
  if (xcdChunk) {
    if ((uint64_t)xcdChunk * kNumXcd < logical) return false;
    blocks = (uint64_t)xcdChunk * kNumXcd;
  }
  return blocks > 0 && blocks <= 0x7fffffffull && blocks * kTileThreads <= CUTT_HIP_MAX_GRID_LANES;
}

// The rows of a tile axis over fused ranks: the extents must multiply to the axis' length.
bool rowRadixOk(const cuttHipRowRadix& rr, int count) {
  if (rr.n == 0) return true;
  if (rr.n < 0 || rr.n > CUTT_MAX_TILE_SET) return false;
  uint64_t vol = 1;
  for (int k = 0; k < rr.n; k++) {
    if (rr.extent[k] < 1 || !divisorOk(rr.div[k], rr.extent[k])) return false;
    vol *= rr.extent[k];
    if (vol > 0x7fffffffull) return false;
  }
  return vol == (uint64_t)count;
}

// Allow dynamic LDS up to the device limit for a kernel (once per process and kernel).
template <typename K>
int allowLargeLds(K kernel, size_t bytes) {
  return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

// ---------------------------------------------------------------------------
// Trivial method: a plain copy, 16 bytes per lane and one 4-KB piece per workgroup, so that the
// hardware dispatcher spreads the pieces and every wave has exactly one load and one store in
// flight.  Measured against the runtime's device-to-device copy: the same below 128 MB, 20-33 %
// faster from 256 MB on with streaming loads (6.4-7.0 against 4.9-5.4 TB/s).
// The last (bytes % 16) / 4 words are copied by the first lanes of workgroup 0.
typedef unsigned int Vec16 __attribute__((ext_vector_type(4)));
constexpr int kCopyThreads = 256;

template <int NT>
__global__ __launch_bounds__(kCopyThreads) void copyKernel(const Vec16* __restrict__ in, Vec16* __restrict__ out,
                                                           uint64_t n16, uint32_t tailWords) {
  const uint64_t i = (uint64_t)blockIdx.x * kCopyThreads + threadIdx.x;
  if (i < n16) stg<NT>(out + i, ldg<NT>(in + i));
  if (blockIdx.x == 0 && threadIdx.x < tailWords) {
    const uint32_t* in32 = (const uint32_t*)(in + n16);
    uint32_t* out32 = (uint32_t*)(out + n16);
    out32[threadIdx.x] = in32[threadIdx.x];
  }
}

}  // namespace

extern "C" int cuttHipPackedRegsPerLaneLoaded(int elemSize, int elemsPerThread, int wideOffsets) {
  const void* f = nullptr;
#define CUTT_PICK(T, E)                                                                       \
  f = wideOffsets ? reinterpret_cast<const void*>(packedKernel<T, E, 0, true>)               \
                  : reinterpret_cast<const void*>(packedKernel<T, E, 0, false>)
  if (elemSize == 4) {
    switch (elemsPerThread) {
      case 1: CUTT_PICK(uint32_t, 1); break;
      case 2: CUTT_PICK(uint32_t, 2); break;
      case 4: CUTT_PICK(uint32_t, 4); break;
      case 8: CUTT_PICK(uint32_t, 8); break;
      case 16: CUTT_PICK(uint32_t, 16); break;
      default: return -1;
    }
  } else if (elemSize == 8) {
    switch (elemsPerThread) {
      case 1: CUTT_PICK(uint64_t, 1); break;
      case 2: CUTT_PICK(uint64_t, 2); break;
      case 4: CUTT_PICK(uint64_t, 4); break;
      case 8: CUTT_PICK(uint64_t, 8); break;
      default: return -1;
    }
  } else {
    return -1;
  }
#undef CUTT_PICK
  hipFuncAttributes attr;
  if (hipFuncGetAttributes(&attr, f) != hipSuccess) return -1;
  return attr.numRegs;
}

namespace {

// A launch reports the launch call's own result.  (hipGetLastError after a launch would also report
// - and clear - an error that an earlier, unrelated call of the application left behind on this
// thread, such as hipErrorNotReady from a stream query.)
template <typename... KArgs, typename... Args>
hipError_t launchKernel(void (*kernel)(KArgs...), dim3 grid, dim3 block, size_t lds, hipStream_t s, Args... args) {
  static_assert(sizeof...(KArgs) == sizeof...(Args), "one argument per kernel parameter");
  std::tuple<std::remove_const_t<KArgs>...> held{args...};
  void* ptrs[sizeof...(KArgs)];
  int i = 0;
  std::apply([&](auto&... v) { ((ptrs[i++] = (void*)&v), ...); }, held);
  return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, lds, s);
}

}  // namespace

extern "C" long long cuttHipTiledGrid(const cuttHipTiledArgs* a) {
  uint64_t blocks = 0;
  if (!a || !tileGrid(a->order, a->tilesM, a->tilesK, a->volMbar, a->xcdChunk, a->superM, a->superK, a->digits, a->mbar, blocks))
    return 0;
  return (long long)blocks;
}

extern "C" long long cuttHipTiledCopyGrid(const cuttHipTiledCopyArgs* a) {
  uint64_t blocks = 0;
  if (!a || !tileGrid(a->order, a->tilesM, a->tilesK, a->volMbar, a->xcdChunk, a->superM, a->superK, a->digits, a->mbar, blocks))
    return 0;
  return (long long)blocks;
}

extern "C" int cuttHipValidateTiled(const cuttHipTiledArgs* a) {
  if (!a) return (int)hipErrorInvalidValue;
  if ((a->elemSize != 4 && a->elemSize != 8) || a->volMm < 1 || a->volMk < 1 || a->volMbar < 1 ||
      a->tilesM != (a->volMm + kTile - 1) / kTile || (a->alignedStores != 0 && a->alignedStores != 1) ||
      a->tilesK != (a->volMk + (a->alignedStores ? 128 / a->elemSize - 1 : 0) + kTile - 1) / kTile ||
      a->order < 0 || a->order > 7 || !mbarOk(a->mbar) || (a->grouped != 0 && a->grouped != 1) ||
      (a->alignedStores && a->grouped) || !rowRadixOk(a->rowsK, a->volMk) || !rowRadixOk(a->rowsM, a->volMm) ||
      (a->alignedStores && (a->rowsK.n > 0 || a->rowsM.n > 0)))
    return (int)hipErrorInvalidValue;
  uint64_t blocks = 0;
  if (!tileGrid(a->order, a->tilesM, a->tilesK, a->volMbar, a->xcdChunk, a->superM, a->superK, a->digits, a->mbar, blocks))
    return (int)hipErrorInvalidConfiguration;
  if (a->cachePolicy != 0 && a->cachePolicy != 1 && a->cachePolicy != 3) return (int)hipErrorInvalidValue;
  return 0;
}

extern "C" int cuttHipLaunchTiled(const cuttHipTiledArgs* a, const void* in, void* out, void* stream) {
  if (!a || !in || !out) return (int)hipErrorInvalidValue;
  uint64_t blocks = 0;
  if (!tileGrid(a->order, a->tilesM, a->tilesK, a->volMbar, a->xcdChunk, a->superM, a->superK, a->digits, a->mbar, blocks))
    return (int)hipErrorInvalidConfiguration;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((uint32_t)blocks), block(kTileThreads);
  const bool fused = a->rowsK.n > 0 || a->rowsM.n > 0;
#define CUTT_LAUNCH_TILED_F(T, NT, G)                                                                            \
  (fused ? launchKernel(tiledKernel<T, NT, G, true>, grid, block, 0, s, *a, (const T*)in, (T*)out)               \
         : launchKernel(tiledKernel<T, NT, G, false>, grid, block, 0, s, *a, (const T*)in, (T*)out))
#define CUTT_LAUNCH_TILED(T, NT)                                                                        \
  return (int)(a->alignedStores                                                                         \
                   ? launchKernel(tiledAlignedKernel<T, NT>, grid, block, 0, s, *a, (const T*)in, (T*)out) \
                   : (a->grouped ? CUTT_LAUNCH_TILED_F(T, NT, true) : CUTT_LAUNCH_TILED_F(T, NT, false)))
#define CUTT_LAUNCH_TILED_NT(T)                                \
  switch (a->cachePolicy) {                                    \
    case 0: CUTT_LAUNCH_TILED(T, 0);                           \
    case 1: CUTT_LAUNCH_TILED(T, 1);                           \
    default: CUTT_LAUNCH_TILED(T, 3);                          \
  }
  if (a->elemSize == 4) {
    CUTT_LAUNCH_TILED_NT(uint32_t)
  } else {
    CUTT_LAUNCH_TILED_NT(uint64_t)
  }
#undef CUTT_LAUNCH_TILED_NT
#undef CUTT_LAUNCH_TILED
#undef CUTT_LAUNCH_TILED_F
}

extern "C" int cuttHipValidateTiledCopy(const cuttHipTiledCopyArgs* a) {
  if (!a) return (int)hipErrorInvalidValue;
  if ((a->elemSize != 4 && a->elemSize != 8) || a->volMm < 1 || a->volMk < 1 || a->volMbar < 1 ||
      a->tilesM != (a->volMm + kTile - 1) / kTile || a->tilesK != (a->volMk + kTile - 1) / kTile ||
      a->order < 0 || a->order > 7 || !mbarOk(a->mbar))
    return (int)hipErrorInvalidValue;
  uint64_t blocks = 0;
  if (!tileGrid(a->order, a->tilesM, a->tilesK, a->volMbar, a->xcdChunk, a->superM, a->superK, a->digits, a->mbar, blocks))
    return (int)hipErrorInvalidConfiguration;
  if (a->cachePolicy != 0 && a->cachePolicy != 1 && a->cachePolicy != 3) return (int)hipErrorInvalidValue;
  return 0;
}

extern "C" int cuttHipLaunchTiledCopy(const cuttHipTiledCopyArgs* a, const void* in, void* out,
                                      void* stream) {
  if (!a || !in || !out) return (int)hipErrorInvalidValue;
  uint64_t blocks = 0;
  if (!tileGrid(a->order, a->tilesM, a->tilesK, a->volMbar, a->xcdChunk, a->superM, a->superK, a->digits, a->mbar, blocks))
    return (int)hipErrorInvalidConfiguration;
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((uint32_t)blocks), block(kTileThreads);
#define CUTT_LAUNCH_TCOPY(T, NT) \
  return (int)launchKernel(tiledCopyKernel<T, NT>, grid, block, 0, s, *a, (const T*)in, (T*)out)
#define CUTT_LAUNCH_TCOPY_NT(T)                                \
  switch (a->cachePolicy) {                                    \
    case 0: CUTT_LAUNCH_TCOPY(T, 0);                           \
    case 1: CUTT_LAUNCH_TCOPY(T, 1);                           \
    default: CUTT_LAUNCH_TCOPY(T, 3);                          \
  }
  if (a->elemSize == 4) {
    CUTT_LAUNCH_TCOPY_NT(uint32_t)
  } else {
    CUTT_LAUNCH_TCOPY_NT(uint64_t)
  }
#undef CUTT_LAUNCH_TCOPY_NT
#undef CUTT_LAUNCH_TCOPY
}

// Plain copy for the Trivial method.  Both pointers 16-byte aligned: copyKernel; otherwise the
// runtime's device-to-device copy.
extern "C" int cuttHipLaunchCopy(const void* in, void* out, size_t bytes, int cachePolicy, void* stream) {
  if (!in || !out || bytes == 0 || bytes % 4 != 0) return (int)hipErrorInvalidValue;
  if (cachePolicy != 0 && cachePolicy != 1 && cachePolicy != 3) return (int)hipErrorInvalidValue;
  hipStream_t s = (hipStream_t)stream;
  if ((((uintptr_t)in | (uintptr_t)out) & 15) != 0)
    return (int)hipMemcpyAsync(out, in, bytes, hipMemcpyDeviceToDevice, s);
  const uint64_t n16 = bytes / 16;
  const uint32_t tailWords = (uint32_t)((bytes % 16) / 4);
  const uint64_t blocks = std::max<uint64_t>(1, (n16 + kCopyThreads - 1) / kCopyThreads);
  if (blocks > 0x7fffffffull || blocks * kCopyThreads > CUTT_HIP_MAX_GRID_LANES) return (int)hipErrorInvalidConfiguration;
  const dim3 grid((uint32_t)blocks), block(kCopyThreads);
  switch (cachePolicy) {
    case 0: return (int)launchKernel(copyKernel<0>, grid, block, 0, s, (const Vec16*)in, (Vec16*)out, n16, tailWords);
    case 1: return (int)launchKernel(copyKernel<1>, grid, block, 0, s, (const Vec16*)in, (Vec16*)out, n16, tailWords);
    default: return (int)launchKernel(copyKernel<3>, grid, block, 0, s, (const Vec16*)in, (Vec16*)out, n16, tailWords);
  }
}

// ---------------------------------------------------------------------------
// Static scratch memory and the kernel that builds a plan's index tables in it.
// ---------------------------------------------------------------------------
// Device memory that exists from the moment the code object is loaded: the entry point that must
// not allocate keeps a packed plan's index tables here.  In host code the array's name is only a
// handle for hipGetSymbolAddress; the address it returns (one per device) is what kernels get.
static __device__ __align__(256) unsigned char scratch[CUTT_HIP_SCRATCH_BYTES];

extern "C" int cuttHipScratch(void** ptr, size_t* bytes) {
  static std::mutex lock;
  static void* perDevice[64] = {};
  if (!ptr || !bytes) return (int)hipErrorInvalidValue;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= 64) return (int)hipErrorInvalidDevice;
  std::lock_guard<std::mutex> guard(lock);
  if (!perDevice[dev]) {
    void* p = nullptr;
    if (hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)); e != hipSuccess) return (int)e;
    if (!p) return (int)hipErrorInvalidSymbol;
    perDevice[dev] = p;
  }
  *ptr = perDevice[dev];
  *bytes = CUTT_HIP_SCRATCH_BYTES;
  return 0;
}

namespace {
constexpr int kBuildThreads = 256;

__device__ __forceinline__ uint32_t radixSum(const cuttHipRadixList& l, uint32_t i) {
  uint32_t off = 0;
  for (int k = 0; k < l.n; k++) {
    const uint32_t q = i / l.extent[k];
    off += (i - q * l.extent[k]) * l.stride[k];
    i = q;
  }
  return off;
}

__global__ __launch_bounds__(kBuildThreads) void buildTablesKernel(const cuttHipTableBuildArgs a) {
  const uint32_t i = blockIdx.x * kBuildThreads + threadIdx.x;
  if (i < a.count[0]) a.rowIn[i] = radixSum(a.list[0], i);
  if (i < a.count[1]) a.rowOut[i] = radixSum(a.list[1], i);
  if (i < a.count[2]) {
    const uint32_t pos = radixSum(a.list[2], i);
    a.shIdx[i] = (uint16_t)(pos + (pos >> a.padShift));
  }
}
}  // namespace

extern "C" int cuttHipLaunchTableBuild(const cuttHipTableBuildArgs* a, void* stream) {
  if (!a || !a->rowIn || !a->rowOut || !a->shIdx || a->padShift < 1 || a->padShift > 31)
    return (int)hipErrorInvalidValue;
  uint32_t most = 0;
  for (int l = 0; l < 3; l++) {
    if (a->count[l] < 1 || a->count[l] > 65536 || a->list[l].n < 0 || a->list[l].n > CUTT_MAX_RANK)
      return (int)hipErrorInvalidValue;
    uint64_t span = 1;  // the list must enumerate at least count entries
    for (int k = 0; k < a->list[l].n; k++) {
      if (a->list[l].extent[k] < 1) return (int)hipErrorInvalidValue;
      span *= a->list[l].extent[k];
      if (span > (1ull << 32)) return (int)hipErrorInvalidValue;
    }
    if (span != a->count[l]) return (int)hipErrorInvalidValue;
    most = std::max(most, a->count[l]);
  }
  const dim3 grid((most + kBuildThreads - 1) / kBuildThreads), block(kBuildThreads);
  return (int)launchKernel(buildTablesKernel, grid, block, 0, (hipStream_t)stream, *a);
}

// Lets the packed kernels use more than the default 64 KB of dynamic LDS on the current device.
// Called when a packed plan is activated, so that every cuttExecute is a plain kernel launch.
extern "C" int cuttHipPreparePacked(void) {
  // Function attributes are kept per device.  Two threads may both find the flag clear and both
  // make the calls: they are idempotent.
  static std::atomic<bool> ldsOptInDone[64];
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return (int)e;
  const bool tracked = dev >= 0 && dev < 64;
  if (!tracked || !ldsOptInDone[dev]) {
    hipDeviceProp_t prop;
    if (hipError_t e = hipGetDeviceProperties(&prop, dev); e != hipSuccess) return (int)e;
    const size_t m = prop.sharedMemPerBlock;
    int r = 0;
#define CUTT_ALLOW(T, E)                                                  \
  if (r == 0) r = allowLargeLds(packedKernel<T, E, 0, false>, m);         \
  if (r == 0) r = allowLargeLds(packedKernel<T, E, 1, false>, m);         \
  if (r == 0) r = allowLargeLds(packedKernel<T, E, 3, false>, m);         \
  if (r == 0) r = allowLargeLds(packedKernel<T, E, 0, true>, m);          \
  if (r == 0) r = allowLargeLds(packedKernel<T, E, 1, true>, m);          \
  if (r == 0) r = allowLargeLds(packedKernel<T, E, 3, true>, m)
    CUTT_ALLOW(uint32_t, 1); CUTT_ALLOW(uint32_t, 2); CUTT_ALLOW(uint32_t, 4); CUTT_ALLOW(uint32_t, 8);
    CUTT_ALLOW(uint32_t, 16);
    CUTT_ALLOW(uint64_t, 1); CUTT_ALLOW(uint64_t, 2); CUTT_ALLOW(uint64_t, 4); CUTT_ALLOW(uint64_t, 8);
#undef CUTT_ALLOW
    if (r != 0) return r;
    if (tracked) ldsOptInDone[dev] = true;
  }
  return 0;
}

// Number of workgroups of a packed launch (0 = the work items do not fit a grid).
static uint64_t packedGrid(const cuttHipPackedArgs* a) {
  const long long items = cuttHipPackedItemNumbers(a);
  if (items < 1) return 0;
  uint64_t blocks = ((uint64_t)items + a->itemsPerBlock - 1) / a->itemsPerBlock;
  if (a->xcdChunk) {
    if ((uint64_t)a->xcdChunk * kNumXcd < blocks) return 0;
    blocks = (uint64_t)a->xcdChunk * kNumXcd;
  }
  return blocks <= 0x7fffffffull && blocks * (uint64_t)a->numThreads <= CUTT_HIP_MAX_GRID_LANES ? blocks : 0;
}

extern "C" int cuttHipValidatePacked(const cuttHipPackedArgs* a) {
  if (!a) return (int)hipErrorInvalidValue;
  if ((a->elemSize != 4 && a->elemSize != 8) || a->numThreads < 64 || a->numThreads > 1024 ||
      (a->numThreads & 63) || a->volMbar < 1 || a->itemsPerBlock < 1 || a->padShift < 1 ||
      a->itemOrder < 0 || a->itemOrder > 2 ||
      (a->elemsPerThread != 1 && a->elemsPerThread != 2 && a->elemsPerThread != 4 &&
       a->elemsPerThread != 8 && !(a->elemsPerThread == 16 && a->elemSize == 4)) ||
      (a->cachePolicy != 0 && a->cachePolicy != 1 && a->cachePolicy != 3) ||
      a->padShift > 31 || a->ldsElems < 1 || a->ldsElems > 65536 || !mbarOk(a->mbar) || a->volume < 1 ||
      a->volume > 0xffffffffll ||
      // 32-bit byte offsets reach 4 GB
      (!a->wideOffsets && (uint64_t)a->volume * (uint64_t)a->elemSize > (1ull << 32)))
    return (int)hipErrorInvalidValue;
  for (int i = 0; i < 2; i++) {
    const cuttHipSplitRank& sr = a->split[i];
    if (sr.numSplit < 1 || sr.slabRem < 0 || sr.slabRem >= sr.numSplit || sr.slabFloor < 0 ||
        !divisorOk(sr.div, (uint32_t)sr.numSplit))
      return (int)hipErrorInvalidValue;
  }
  for (int c = 0; c < 4; c++) {
    // class c is used only if the split ranks it refers to have slabs of the larger size
    if (((c & 1) && a->split[0].slabRem == 0) || ((c & 2) && a->split[1].slabRem == 0)) continue;
    const cuttHipPackedClass& k = a->cls[c];
    if (k.vol < 1 || k.vol > a->maxVol || (int64_t)a->numThreads * a->elemsPerThread < k.vol || !k.rowIn ||
        !k.rowOut || !k.shIdx || k.inCont < 1 || k.outCont < 1 || k.vol % k.inCont || k.vol % k.outCont ||
        !divisorOk(k.inDiv, (uint32_t)k.inCont) || !divisorOk(k.outDiv, (uint32_t)k.outCont))
      return (int)hipErrorInvalidValue;
    const uint32_t last = (uint32_t)k.vol - 1;
    if ((int)(last + (last >> a->padShift)) >= a->ldsElems) return (int)hipErrorInvalidValue;
  }
  if (packedGrid(a) == 0) return (int)hipErrorInvalidConfiguration;
  return 0;
}

extern "C" int cuttHipLaunchPacked(const cuttHipPackedArgs* a, const void* in, void* out, void* stream) {
  if (!a || !in || !out) return (int)hipErrorInvalidValue;
  const uint64_t blocks = packedGrid(a);
  if (blocks == 0) return (int)hipErrorInvalidConfiguration;
  const size_t lds = cuttHipPackedLdsBytes(a);
  hipStream_t s = (hipStream_t)stream;
  const dim3 grid((uint32_t)blocks), block(a->numThreads);
  const bool wide = a->wideOffsets != 0;
#define CUTT_LAUNCH_PACKED(T, E, NT)                                                                              \
  return (int)(wide ? launchKernel(packedKernel<T, E, NT, true>, grid, block, lds, s, *a, (const T*)in, (T*)out)  \
                    : launchKernel(packedKernel<T, E, NT, false>, grid, block, lds, s, *a, (const T*)in, (T*)out))
#define CUTT_LAUNCH_PACKED_NT(T, E)                            \
  switch (a->cachePolicy) {                                    \
    case 0: CUTT_LAUNCH_PACKED(T, E, 0);                       \
    case 1: CUTT_LAUNCH_PACKED(T, E, 1);                       \
    default: CUTT_LAUNCH_PACKED(T, E, 3);                      \
  }
#define CUTT_LAUNCH_PACKED_E(T)                                \
  switch (a->elemsPerThread) {                                 \
    case 1: CUTT_LAUNCH_PACKED_NT(T, 1)                        \
    case 2: CUTT_LAUNCH_PACKED_NT(T, 2)                        \
    case 4: CUTT_LAUNCH_PACKED_NT(T, 4)                        \
    default: CUTT_LAUNCH_PACKED_NT(T, 8)                       \
  }
  if (a->elemSize == 4 && a->elemsPerThread == 16) {
    // 4-byte elements only: 16 per lane stage the same 64 KB as 8 per lane do for 8-byte elements
    CUTT_LAUNCH_PACKED_NT(uint32_t, 16)
  } else if (a->elemSize == 4) {
    CUTT_LAUNCH_PACKED_E(uint32_t)
  } else {
    CUTT_LAUNCH_PACKED_E(uint64_t)
  }
#undef CUTT_LAUNCH_PACKED_NT
#undef CUTT_LAUNCH_PACKED_E
#undef CUTT_LAUNCH_PACKED
}
