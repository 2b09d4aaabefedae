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
 *  - the per-rank decomposition of a workgroup's Mbar position is wave-uniform
 *    and read from the kernel-argument segment (scalar loads), instead of
 *    one-table-entry-per-lane plus cross-lane shuffles;
 *  - Tiled stages a 64x64 tile in LDS padded to 65 columns (conflict-free for
 *    both 4- and 8-byte words); each lane keeps 16 loads in flight;
 *  - Packed/PackedSplit keep their index-remap tables in LDS: a u16 gather
 *    index per element plus one offset per contiguous row, with the
 *    row/column split done by a multiply-high; the LDS data buffer is skewed
 *    by one slot per 2^padShift to break power-of-two bank strides;
 *  - workgroups are short-lived and small (a tile, or a few Mbar positions),
 *    thousands are in flight: on this chip that streams faster than a
 *    persistent grid-stride loop.
 *
 * All offsets are 32-bit element offsets (the API limits a tensor to fewer
 * than 2^31 elements); they are widened only when added to the base pointer.
 */
#include <hip/hip_runtime.h>

#include "hip_layer.h"

namespace {

constexpr int kTile = 64;             // tile edge in elements
constexpr int kTileThreads = 256;     // 4 wavefronts
constexpr int kTileRows = kTile * kTile / kTileThreads;  // rows per lane: 16
constexpr int kWaves = kTileThreads / 64;

// Decompose Mbar position m (wave-uniform) into input and output offsets.
__device__ __forceinline__ void mbarOffsets(const cuttHipMbar& mb, uint32_t m, uint32_t& offIn,
                                            uint32_t& offOut) {
  uint32_t oi = 0, oo = 0;
  for (int k = 0; k < mb.n; k++) {
    const uint32_t e = mb.d[k].extent;
    const uint32_t q = m / e;
    const uint32_t i = m - q * e;
    oi += i * mb.d[k].strideIn;
    oo += i * mb.d[k].strideOut;
    m = q;
  }
  offIn = oi;
  offOut = oo;
}

// Workgroup index -> (tile along Mm, tile along Mk, Mbar position).
__device__ __forceinline__ void decodeTile(uint32_t bid, int order, uint32_t tilesM, uint32_t tilesK,
                                           uint32_t volMbar, uint32_t& tm, uint32_t& tk, uint32_t& m) {
  if (order == 0) {
    const uint32_t t = bid / volMbar;
    m = bid - t * volMbar;
    tk = t / tilesM;
    tm = t - tk * tilesM;
  } else if (order == 1) {
    const uint32_t t = bid / tilesM;
    tm = bid - t * tilesM;
    m = t / tilesK;
    tk = t - m * tilesK;
  } else {
    const uint32_t t = bid / tilesK;
    tk = bid - t * tilesK;
    m = t / tilesM;
    tm = t - m * tilesM;
  }
}

// ---------------------------------------------------------------------------
// Tiled: 64x64 tile through padded LDS.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kTileThreads) void tiledKernel(const cuttHipTiledArgs a,
                                                            const T* __restrict__ in,
                                                            T* __restrict__ out) {
  __shared__ T tile[kTile][kTile + 1];

  uint32_t tm, tk, m;
  decodeTile(blockIdx.x, a.order, a.tilesM, a.tilesK, a.volMbar, tm, tk, m);
  uint32_t offIn, offOut;
  mbarOffsets(a.mbar, m, offIn, offOut);

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t m0 = tm * kTile, k0 = tk * kTile;
  const uint32_t volMm = a.volMm, volMk = a.volMk;

  // Read: lanes run along input rank 0, rows along the Mk rank.
  {
    const uint32_t x = m0 + lane;
    const bool xok = x < volMm;
    T v[kTileRows];
#pragma unroll
    for (int j = 0; j < kTileRows; j++) {
      const uint32_t r = wave + kWaves * j;
      const uint32_t k = k0 + r;
      if (xok && k < volMk) v[j] = in[offIn + x + k * a.strideInK];
    }
#pragma unroll
    for (int j = 0; j < kTileRows; j++) {
      const uint32_t r = wave + kWaves * j;
      if (xok && k0 + r < volMk) tile[r][lane] = v[j];
    }
  }
  __syncthreads();
  // Write: lanes run along the Mk rank (contiguous in the output).
  {
    const uint32_t k = k0 + lane;
    const bool kok = k < volMk;
#pragma unroll
    for (int j = 0; j < kTileRows; j++) {
      const uint32_t r = wave + kWaves * j;
      const uint32_t x = m0 + r;
      if (kok && x < volMm) out[offOut + k + x * a.strideOutM] = tile[lane][r];
    }
  }
}

// ---------------------------------------------------------------------------
// TiledCopy: rank 0 stays in front; rows are copied through registers.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(kTileThreads) void tiledCopyKernel(const cuttHipTiledCopyArgs a,
                                                                const T* __restrict__ in,
                                                                T* __restrict__ out) {
  uint32_t tm, tk, m;
  decodeTile(blockIdx.x, a.order, a.tilesM, a.tilesK, a.volMbar, tm, tk, m);
  uint32_t offIn, offOut;
  mbarOffsets(a.mbar, m, offIn, offOut);

  const uint32_t lane = threadIdx.x & 63;
  const uint32_t wave = threadIdx.x >> 6;
  const uint32_t x = tm * kTile + lane;
  const uint32_t k0 = tk * kTile;
  const bool xok = x < (uint32_t)a.volMm;
  const uint32_t volMk = a.volMk;

  T v[kTileRows];
#pragma unroll
  for (int j = 0; j < kTileRows; j++) {
    const uint32_t k = k0 + wave + kWaves * j;
    if (xok && k < volMk) v[j] = in[offIn + x + k * a.strideInK];
  }
#pragma unroll
  for (int j = 0; j < kTileRows; j++) {
    const uint32_t k = k0 + wave + kWaves * j;
    if (xok && k < volMk) out[offOut + x + k * a.strideOutK] = v[j];
  }
}

// ---------------------------------------------------------------------------
// Packed / PackedSplit: stage a block of Mmk through LDS with remap tables.
// ---------------------------------------------------------------------------
constexpr int kPackedUnroll = 4;

// n / d for n < 2^16, 2 <= d <= 2^16 with magic = ceil(2^32 / d); d == 1 handled apart.
__device__ __forceinline__ uint32_t divSmall(uint32_t n, uint32_t d, uint32_t magic) {
  return d == 1 ? n : __umulhi(n, magic);
}

template <typename T>
__global__ void packedKernel(const cuttHipPackedArgs a, const T* __restrict__ in,
                             T* __restrict__ out) {
  extern __shared__ __align__(16) unsigned char ldsRaw[];
  T* buf = reinterpret_cast<T*>(ldsRaw);
  uint32_t* sRowIn = reinterpret_cast<uint32_t*>(buf + a.ldsElems);
  uint32_t* sRowOut = sRowIn + a.maxRowsIn;
  uint16_t* sSh = reinterpret_cast<uint16_t*>(sRowOut + a.maxRowsOut);

  const uint32_t tid = threadIdx.x;
  const uint32_t nt = blockDim.x;
  const uint32_t numSplit = a.numSplit;
  const uint32_t totalItems = (uint32_t)a.volMbar * numSplit;
  const uint32_t w0 = blockIdx.x * (uint32_t)a.itemsPerBlock;
  const uint32_t w1 = min(w0 + (uint32_t)a.itemsPerBlock, totalItems);
  const uint32_t slabRem = a.slabRem;
  const int padShift = a.padShift;

  int loaded = -1;
  for (uint32_t w = w0; w < w1; w++) {
    const uint32_t m = w / numSplit;
    const uint32_t s = w - m * numSplit;
    const int c = (s < slabRem) ? 1 : 0;
    const uint32_t p0 = s * (uint32_t)a.slabFloor + min(s, slabRem);

    uint32_t offIn, offOut;
    mbarOffsets(a.mbar, m, offIn, offOut);
    offIn += p0 * a.splitStrideIn;
    offOut += p0 * a.splitStrideOut;

    const uint32_t vol = a.cls[c].vol;
    const uint32_t inCont = a.cls[c].inCont, outCont = a.cls[c].outCont;
    const uint32_t inMagic = a.cls[c].inMagic, outMagic = a.cls[c].outMagic;

    __syncthreads();  // the previous item has finished reading the LDS buffer
    if (c != loaded) {
      const uint32_t nIn = a.cls[c].nRowsIn, nOut = a.cls[c].nRowsOut;
      const uint32_t* gIn = a.cls[c].rowIn;
      const uint32_t* gOut = a.cls[c].rowOut;
      const uint16_t* gSh = a.cls[c].shIdx;
      for (uint32_t i = tid; i < nIn; i += nt) sRowIn[i] = gIn[i];
      for (uint32_t i = tid; i < nOut; i += nt) sRowOut[i] = gOut[i];
      for (uint32_t i = tid; i < vol; i += nt) sSh[i] = gSh[i];
      loaded = c;
      __syncthreads();
    }

    // Global -> LDS in input-compact order.
    for (uint32_t base = tid; base < vol; base += nt * kPackedUnroll) {
      T v[kPackedUnroll];
#pragma unroll
      for (int u = 0; u < kPackedUnroll; u++) {
        const uint32_t p = base + u * nt;
        if (p < vol) {
          const uint32_t row = divSmall(p, inCont, inMagic);
          const uint32_t col = p - row * inCont;
          v[u] = in[offIn + sRowIn[row] + col];
        }
      }
#pragma unroll
      for (int u = 0; u < kPackedUnroll; u++) {
        const uint32_t p = base + u * nt;
        if (p < vol) buf[p + (p >> padShift)] = v[u];
      }
    }
    __syncthreads();
    // LDS -> global in output-compact order.
    for (uint32_t base = tid; base < vol; base += nt * kPackedUnroll) {
#pragma unroll
      for (int u = 0; u < kPackedUnroll; u++) {
        const uint32_t q = base + u * nt;
        if (q < vol) {
          const uint32_t row = divSmall(q, outCont, outMagic);
          const uint32_t col = q - row * outCont;
          out[offOut + sRowOut[row] + col] = buf[sSh[q]];
        }
      }
    }
  }
}

size_t packedLdsBytes(const cuttHipPackedArgs* a) {
  size_t b = (size_t)a->ldsElems * a->elemSize;
  b += sizeof(uint32_t) * ((size_t)a->maxRowsIn + a->maxRowsOut);
  b += sizeof(uint16_t) * (size_t)a->maxVol;
  return (b + 15) & ~(size_t)15;
}

bool mbarOk(const cuttHipMbar& mb) {
  if (mb.n < 0 || mb.n > CUTT_MAX_RANK) return false;
  for (int k = 0; k < mb.n; k++)
    if (mb.d[k].extent == 0) return false;
  return true;
}

// Allow dynamic LDS up to the device limit for a kernel (once per process and kernel).
template <typename K>
int allowLargeLds(K kernel, size_t bytes) {
  return (int)hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
}

}  // namespace

extern "C" size_t cuttHipPackedLdsBytes(const cuttHipPackedArgs* a) { return packedLdsBytes(a); }

extern "C" int cuttHipLaunchTiled(const cuttHipTiledArgs* a, const void* in, void* out, void* stream) {
  if (!a || !in || !out) return (int)hipErrorInvalidValue;
  if ((a->elemSize != 4 && a->elemSize != 8) || a->volMm < 1 || a->volMk < 1 || a->volMbar < 1 ||
      a->tilesM != (a->volMm + kTile - 1) / kTile || a->tilesK != (a->volMk + kTile - 1) / kTile ||
      a->order < 0 || a->order > 2 || !mbarOk(a->mbar))
    return (int)hipErrorInvalidValue;
  const uint64_t blocks = (uint64_t)a->tilesM * a->tilesK * (uint64_t)a->volMbar;
  if (blocks == 0 || blocks > 0x7fffffffull) return (int)hipErrorInvalidConfiguration;
  hipStream_t s = (hipStream_t)stream;
  if (a->elemSize == 4)
    hipLaunchKernelGGL(tiledKernel<uint32_t>, dim3((uint32_t)blocks), dim3(kTileThreads), 0, s, *a,
                       (const uint32_t*)in, (uint32_t*)out);
  else
    hipLaunchKernelGGL(tiledKernel<uint64_t>, dim3((uint32_t)blocks), dim3(kTileThreads), 0, s, *a,
                       (const uint64_t*)in, (uint64_t*)out);
  return (int)hipGetLastError();
}

extern "C" int cuttHipLaunchTiledCopy(const cuttHipTiledCopyArgs* a, const void* in, void* out,
                                      void* stream) {
  if (!a || !in || !out) return (int)hipErrorInvalidValue;
  if ((a->elemSize != 4 && a->elemSize != 8) || a->volMm < 1 || a->volMk < 1 || a->volMbar < 1 ||
      a->tilesM != (a->volMm + kTile - 1) / kTile || a->tilesK != (a->volMk + kTile - 1) / kTile ||
      a->order < 0 || a->order > 2 || !mbarOk(a->mbar))
    return (int)hipErrorInvalidValue;
  const uint64_t blocks = (uint64_t)a->tilesM * a->tilesK * (uint64_t)a->volMbar;
  if (blocks == 0 || blocks > 0x7fffffffull) return (int)hipErrorInvalidConfiguration;
  hipStream_t s = (hipStream_t)stream;
  if (a->elemSize == 4)
    hipLaunchKernelGGL(tiledCopyKernel<uint32_t>, dim3((uint32_t)blocks), dim3(kTileThreads), 0, s, *a,
                       (const uint32_t*)in, (uint32_t*)out);
  else
    hipLaunchKernelGGL(tiledCopyKernel<uint64_t>, dim3((uint32_t)blocks), dim3(kTileThreads), 0, s, *a,
                       (const uint64_t*)in, (uint64_t*)out);
  return (int)hipGetLastError();
}

extern "C" int cuttHipLaunchPacked(const cuttHipPackedArgs* a, const void* in, void* out, void* stream) {
  if (!a || !in || !out) return (int)hipErrorInvalidValue;
  if ((a->elemSize != 4 && a->elemSize != 8) || a->numThreads < 64 || a->numThreads > 1024 ||
      (a->numThreads & 63) || a->volMbar < 1 || a->numSplit < 1 || a->itemsPerBlock < 1 ||
      a->slabRem < 0 || a->slabRem >= a->numSplit || a->padShift < 1 || a->padShift > 31 ||
      a->ldsElems < 1 || a->ldsElems > 65536 || !mbarOk(a->mbar))
    return (int)hipErrorInvalidValue;
  const int ncls = (a->slabRem > 0) ? 2 : 1;
  for (int c = 0; c < ncls; c++) {
    const cuttHipPackedClass& k = a->cls[c];
    if (k.vol < 1 || k.vol > a->maxVol || k.inCont < 1 || k.outCont < 1 || k.nRowsIn > a->maxRowsIn ||
        k.nRowsOut > a->maxRowsOut || (int64_t)k.nRowsIn * k.inCont != k.vol ||
        (int64_t)k.nRowsOut * k.outCont != k.vol || !k.rowIn || !k.rowOut || !k.shIdx)
      return (int)hipErrorInvalidValue;
    const uint32_t last = (uint32_t)k.vol - 1;
    if ((int)(last + (last >> a->padShift)) >= a->ldsElems) return (int)hipErrorInvalidValue;
  }
  const uint64_t items = (uint64_t)a->volMbar * a->numSplit;
  const uint64_t blocks = (items + a->itemsPerBlock - 1) / a->itemsPerBlock;
  if (items > 0x7fffffffull || blocks == 0) return (int)hipErrorInvalidConfiguration;
  const size_t lds = packedLdsBytes(a);

  static bool ldsOptIn = false;  // benign if two threads race: the call is idempotent
  if (!ldsOptIn) {
    int dev = 0;
    hipDeviceProp_t prop;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess) e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return (int)e;
    int r = allowLargeLds(packedKernel<uint32_t>, prop.sharedMemPerBlock);
    if (r == 0) r = allowLargeLds(packedKernel<uint64_t>, prop.sharedMemPerBlock);
    if (r != 0) return r;
    ldsOptIn = true;
  }
  hipStream_t s = (hipStream_t)stream;
  if (a->elemSize == 4)
    hipLaunchKernelGGL(packedKernel<uint32_t>, dim3((uint32_t)blocks), dim3(a->numThreads), lds, s, *a,
                       (const uint32_t*)in, (uint32_t*)out);
  else
    hipLaunchKernelGGL(packedKernel<uint64_t>, dim3((uint32_t)blocks), dim3(a->numThreads), lds, s, *a,
                       (const uint64_t*)in, (uint64_t*)out);
  return (int)hipGetLastError();
}
