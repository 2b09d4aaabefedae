/*
 * count_kernels.hip - kernels that replay the address streams of the transpose kernels and count
 * what the cost model counts on the host: wavefront-level memory instructions, the 128-byte lines
 * and 32-byte sectors each of them touches, partly written lines, LDS bank-conflict degrees.
 *
 * They take the same arguments and the same grid as the kernel they mirror and derive every
 * address with the device functions that kernel itself calls (tile_order.h: tile order, tile geometry and
 * row addresses; packed_items.h: work-item orders, item offsets, run tables; mbar_decode.h), but issue
 * no load or store of tensor data (the instance of the Tiled kernel with line-aligned stores has no
 * counting kernel: cuttHipCountTiled refuses it); the counts of all wavefronts are added up
 * with atomics.  A test compares them with the host model's walk over the same plan.  Counterpart
 * of the reference's model-validation kernels (src/cuttGpuModelKernel.cu:246-646, countTiled,
 * countPacked, countPackedSplit, countTiledCopy, and the driver :686-782), redone for 64-lane
 * wavefronts: distinct lines of a request are counted with 64-bit ballots.
 *
 * Definitions (the host model's, model.cpp):
 *  - an instruction is one wavefront-wide load or store; it is "idle" when every lane only repeats
 *    an edge element (the kernels clamp indices instead of branching); idle instructions are
 *    counted apart and contribute no lines;
 *  - lines / sectors of an instruction: distinct 128-byte / 32-byte blocks among its lanes'
 *    addresses, taking element offsets as byte offsets from a 128-byte aligned buffer;
 *  - partly written lines: per contiguous output run of a work item, one for a head and one for a
 *    tail that does not end on a line boundary (one if the run lies inside a single line);
 *  - LDS cycles of the packed kernel: per gather instruction, conflict degree * words + words,
 *    degree = most lanes on one of 64 four-byte banks (an 8-byte word counted on its first bank).
 */
#include <hip/hip_runtime.h>

#include <tuple>
#include <type_traits>

#include "hip_layer.h"
#include "mbar_decode.h"
#include "packed_items.h"
#include "tile_order.h"

using namespace cutt;

namespace {

enum { kRdInstr, kWrInstr, kRdIdle, kWrIdle, kRdLines, kWrLines, kRdSectors, kWrSectors, kWrPartial, kLdsCycles, kNumCounts };

struct LaneCounts {
  unsigned long long v[kNumCounts];
  unsigned int maxDegree;
};

// Number of distinct values of `key` over the 64 lanes (all lanes active).
__device__ __forceinline__ uint32_t waveDistinct(uint64_t key) {
  uint64_t todo = ~0ull;
  uint32_t n = 0;
  const uint32_t lane = threadIdx.x & 63;
  while (todo) {
    const int first = __ffsll((long long)todo) - 1;
    const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)key, first);
    const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(key >> 32), first);
    const uint64_t same = __ballot(key == (((uint64_t)hi << 32) | lo));
    todo &= ~same;
    n++;
  }
  (void)lane;
  return n;
}

// Largest number of lanes with the same value of `bank` (0..63) among the lanes in `own` (lanes
// that repeat an edge element's slot add to no bank of their own).
__device__ __forceinline__ uint32_t waveMaxMultiplicity(uint32_t bank, uint64_t own) {
  uint64_t todo = own;
  uint32_t most = 0;
  while (todo) {
    const int first = __ffsll((long long)todo) - 1;
    const uint32_t b = (uint32_t)__builtin_amdgcn_readlane((int)bank, first);
    const uint64_t same = __ballot(bank == b) & own;
    todo &= ~same;
    most = max(most, (uint32_t)__popcll(same));
  }
  return most;
}

// Partly covered lines at the two ends of the run of n elements that starts at element `pos`.
__device__ __forceinline__ uint32_t partialEnds(uint64_t pos, uint32_t n, uint32_t es) {
  const uint64_t b0 = pos * es, b1 = (pos + n) * es;
  const bool head = (b0 & 127) != 0, tail = (b1 & 127) != 0;
  if ((b0 >> 7) == ((b1 - 1) >> 7)) return (head || tail) ? 1u : 0u;
  return (uint32_t)head + (uint32_t)tail;
}

// Adds a wavefront's counts (held by lane 0) to the totals.
__device__ __forceinline__ void flush(const LaneCounts& c, unsigned long long* total) {
  if ((threadIdx.x & 63) != 0) return;
  for (int i = 0; i < kNumCounts; i++)
    if (c.v[i]) atomicAdd(&total[i], c.v[i]);
  atomicMax((unsigned int*)&total[kNumCounts], c.maxDegree);
}

// One global-memory instruction of a wavefront: `elem` is every lane's element offset.
__device__ __forceinline__ void countAccess(LaneCounts& c, bool write, bool idle, uint64_t elem, uint32_t es) {
  if (idle) {
    c.v[write ? kWrIdle : kRdIdle] += 1;
    return;
  }
  const uint64_t byte = elem * es;
  c.v[write ? kWrInstr : kRdInstr] += 1;
  c.v[write ? kWrLines : kRdLines] += waveDistinct(byte >> 7);
  c.v[write ? kWrSectors : kRdSectors] += waveDistinct(byte >> 5);
}

// Mirrors tiledKernel: the tile order, the Mbar decode and the lanes' row addresses come from the
// functions that kernel uses (tile_order.h: decodeTile, tileLanes, tileReadElem, tileWriteElem).
template <bool FUSED>
__global__ __launch_bounds__(kTileThreads) void countTiledKernel(const cuttHipTiledArgs a, unsigned long long* total) {
  uint32_t tm, tk, offIn, offOut;
  if (!locateTile(a, tm, tk, offIn, offOut)) return;
  const uint32_t es = (uint32_t)a.elemSize, words = es / 4;
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const TileLanes t = tileLanes<FUSED>(a, tm, tk, offIn, offOut, lane, wave);
  LaneCounts c = {};
  // reads: lanes along the input-contiguous axis, rows along Mk
  for (int j = 0; j < kTileRows; j++) {
    if ((uint32_t)(j / kGroupRows) >= t.groupsK) continue;
    const uint32_t row = wave + kWaves * j, r = min(row, t.wK);
    countAccess(c, false, row > t.wK, tileReadElem<FUSED>(t, a, wave, j), es);
    if (row <= t.wK) c.maxDegree = max(c.maxDegree, waveMaxMultiplicity(((r * (kTile + 1) + t.cx) * words) & 63, __ballot(lane <= t.wM)));
  }
  // writes: lanes along the output-contiguous axis, rows along Mm
  for (int j = 0; j < kTileRows; j++) {
    if ((uint32_t)(j / kGroupRows) >= t.groupsM) continue;
    const uint32_t row = wave + kWaves * j, r = min(row, t.wM);
    const uint32_t elem = tileWriteElem<FUSED>(t, a, wave, j);
    countAccess(c, true, row > t.wM, elem, es);
    if (row <= t.wM) c.maxDegree = max(c.maxDegree, waveMaxMultiplicity(((t.ck * (kTile + 1) + r) * words) & 63, __ballot(lane <= t.wK)));
    // lane 0 holds the first element of the row's run inside this tile
    if (row <= t.wM && lane == 0) c.v[kWrPartial] += partialEnds(elem, t.wK + 1, es);
  }
  // the partial-line counts sit in lane 0 already; the per-instruction counts are wave-uniform
  flush(c, total);
}

// Mirrors tiledCopyKernel (its whole address arithmetic is the three lines below).
__global__ __launch_bounds__(kTileThreads) void countTiledCopyKernel(const cuttHipTiledCopyArgs a, unsigned long long* total) {
  uint32_t tm, tk, offIn, offOut;
  if (!locateTile(a, tm, tk, offIn, offOut)) return;
  const uint32_t es = (uint32_t)a.elemSize;
  const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const uint32_t m0 = tm * kTile, k0 = tk * kTile;
  const uint32_t wM = min((uint32_t)kTile, (uint32_t)a.volMm - m0) - 1;
  const uint32_t wK = min((uint32_t)kTile, (uint32_t)a.volMk - k0) - 1;
  const uint32_t groupsK = (wK >> 4) + 1;
  const uint32_t cx = min(lane, wM);
  LaneCounts c = {};
  for (int j = 0; j < kTileRows; j++) {
    if ((uint32_t)(j / kGroupRows) >= groupsK) continue;
    const uint32_t row = wave + kWaves * j, r = min(row, wK);
    countAccess(c, false, row > wK, (uint64_t)offIn + m0 + cx + (uint64_t)(k0 + r) * a.strideInK, es);
  }
  for (int j = 0; j < kTileRows; j++) {
    if ((uint32_t)(j / kGroupRows) >= groupsK) continue;
    const uint32_t row = wave + kWaves * j, r = min(row, wK);
    const uint64_t start = (uint64_t)offOut + m0 + (uint64_t)(k0 + r) * a.strideOutK;
    countAccess(c, true, row > wK, start + cx, es);
    if (row <= wK && lane == 0) c.v[kWrPartial] += partialEnds(start, wM + 1, es);
  }
  flush(c, total);
}

// Mirrors packedKernel: the work items a workgroup takes and where they lie (all three work-item
// orders), and the lanes' offsets inside a staged block, come from the functions that kernel uses
// (packed_items.h: packedItems, packedLocate, packedInElem, packedOutElem); E elements per lane.
__global__ __launch_bounds__(1024) void countPackedKernel(const cuttHipPackedArgs a, unsigned long long* total) {
  const uint32_t tid = threadIdx.x, nt = blockDim.x, lane = tid & 63;
  const uint32_t es = (uint32_t)a.elemSize, words = es / 4;
  const uint32_t E = (uint32_t)a.elemsPerThread;
  const PackedItems items = packedItems(a);
  const MbarLane mbarLane = loadMbarLane(a.mbar, lane);
  LaneCounts c = {};
  for (uint32_t w = 0; w < items.count; w++) {
    int cls;
    uint32_t offIn, offOut;
    packedLocate(a, items, mbarLane, w, cls, offIn, offOut);
    const cuttHipPackedClass& k = a.cls[cls];
    const uint32_t last = (uint32_t)k.vol - 1;
    for (uint32_t j = 0; j < E; j++) {
      const uint32_t pRaw = tid + j * nt, p = min(pRaw, last);
      const bool idle = pRaw - lane > last;  // the wavefront's first lane is already beyond the block
      countAccess(c, false, idle, (uint64_t)offIn + packedInElem(k, p), es);
      const uint32_t out = packedOutElem(k, p);
      const uint32_t ro = fastDivide(p, k.outDiv.mul, k.outDiv.shift, k.outDiv.add);
      const uint32_t col = p - ro * (uint32_t)k.outCont;
      countAccess(c, true, idle, (uint64_t)offOut + out, es);
      if (!idle) {
        // lanes beyond the block repeat the last element's slot: they add to no bank of their own
        const uint32_t bank = ((uint32_t)k.shIdx[p] * words) & 63;
        const uint32_t degree = waveMaxMultiplicity(bank, __ballot(pRaw <= last));
        c.v[kLdsCycles] += (unsigned long long)degree * words + words;
        c.maxDegree = max(c.maxDegree, degree);
      }
      // every lane that holds the first element of an output run accounts for the run's two ends
      uint32_t ends = (pRaw <= last && col == 0) ? partialEnds((uint64_t)offOut + out, (uint32_t)k.outCont, es) : 0u;
      for (int off = 32; off >= 1; off >>= 1) ends += __shfl_xor(ends, off);
      c.v[kWrPartial] += ends;
    }
  }
  flush(c, total);
}

template <typename... KArgs, typename... Args>
hipError_t launchCount(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t s, Args... args) {
  std::tuple<std::remove_const_t<KArgs>...> held{args...};
  void* ptrs[sizeof...(KArgs)];
  int i = 0;
  std::apply([&](auto&... v) { ((ptrs[i++] = (void*)&v), ...); }, held);
  return hipLaunchKernel(reinterpret_cast<const void*>(kernel), grid, block, ptrs, 0, s);
}

// Runs `launch(totals)` on device totals that start at zero and copies them into `out`.
template <class F>
int runCount(cuttHipStreamCounts* out, void* stream, F&& launch) {
  if (!out) return (int)hipErrorInvalidValue;
  unsigned long long* d = nullptr;
  const size_t bytes = (kNumCounts + 1) * sizeof(unsigned long long);
  if (hipError_t e = hipMalloc((void**)&d, bytes); e != hipSuccess) return (int)e;
  hipStream_t s = (hipStream_t)stream;
  unsigned long long h[kNumCounts + 1] = {};
  hipError_t e = hipMemsetAsync(d, 0, bytes, s);
  if (e == hipSuccess) e = launch(d, s);
  if (e == hipSuccess) e = hipMemcpyAsync(h, d, bytes, hipMemcpyDeviceToHost, s);
  if (e == hipSuccess) e = hipStreamSynchronize(s);
  (void)hipFree(d);
  if (e != hipSuccess) return (int)e;
  out->rdInstr = h[kRdInstr]; out->wrInstr = h[kWrInstr];
  out->rdInstrIdle = h[kRdIdle]; out->wrInstrIdle = h[kWrIdle];
  out->rdLines = h[kRdLines]; out->wrLines = h[kWrLines];
  out->rdSectors = h[kRdSectors]; out->wrSectors = h[kWrSectors];
  out->wrPartialLines = h[kWrPartial]; out->ldsCycles = h[kLdsCycles];
  out->ldsMaxDegree = (unsigned int)h[kNumCounts];
  return 0;
}

}  // namespace

extern "C" int cuttHipCountTiled(const cuttHipTiledArgs* a, cuttHipStreamCounts* out, void* stream) {
  if (int v = cuttHipValidateTiled(a); v != 0) return v;
  if (a->alignedStores) return (int)hipErrorNotSupported;
  const long long blocks = cuttHipTiledGrid(a);
  if (blocks < 1) return (int)hipErrorInvalidConfiguration;
  const bool fused = a->rowsK.n > 0 || a->rowsM.n > 0;
  return runCount(out, stream, [&](unsigned long long* d, hipStream_t s) {
    return fused ? launchCount(countTiledKernel<true>, dim3((uint32_t)blocks), dim3(kTileThreads), s, *a, d)
                 : launchCount(countTiledKernel<false>, dim3((uint32_t)blocks), dim3(kTileThreads), s, *a, d);
  });
}

extern "C" int cuttHipCountTiledCopy(const cuttHipTiledCopyArgs* a, cuttHipStreamCounts* out, void* stream) {
  if (int v = cuttHipValidateTiledCopy(a); v != 0) return v;
  const long long blocks = cuttHipTiledCopyGrid(a);
  if (blocks < 1) return (int)hipErrorInvalidConfiguration;
  return runCount(out, stream, [&](unsigned long long* d, hipStream_t s) {
    return launchCount(countTiledCopyKernel, dim3((uint32_t)blocks), dim3(kTileThreads), s, *a, d);
  });
}

extern "C" int cuttHipCountPacked(const cuttHipPackedArgs* a, cuttHipStreamCounts* out, void* stream) {
  if (int v = cuttHipValidatePacked(a); v != 0) return v;
  const long long numbers = cuttHipPackedItemNumbers(a);
  if (numbers < 1) return (int)hipErrorInvalidConfiguration;
  uint64_t blocks = ((uint64_t)numbers + a->itemsPerBlock - 1) / a->itemsPerBlock;
  if (a->xcdChunk) blocks = (uint64_t)a->xcdChunk * kNumXcd;
  return runCount(out, stream, [&](unsigned long long* d, hipStream_t s) {
    return launchCount(countPackedKernel, dim3((uint32_t)blocks), dim3(a->numThreads), s, *a, d);
  });
}
