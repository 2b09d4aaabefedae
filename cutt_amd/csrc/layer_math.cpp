/*
 * layer_math.cpp - the part of the C-ABI layer (hip_layer.h) that is plain arithmetic: division
 * constants, the Mbar table's derived fields, LDS bytes and register counts of the packed kernel.
 * No HIP header and no runtime call, so the host planner can be linked and tested without the
 * device side (the kernels check their arguments with the same functions).
 */
#include "hip_layer.h"

extern "C" cuttHipDivisor cuttHipMakeDivisor(uint32_t d) {
  cuttHipDivisor dv = {0u, 0u, 1u};  // d <= 1: n / 1
  if (d >= 2) {
    uint32_t shift = 0;
    while ((1ull << (shift + 1)) < d) shift++;  // ceil(log2 d) - 1
    const uint64_t pow2 = 1ull << (32 + shift);
    dv.mul = (uint32_t)((pow2 + d - 1) / d);
    dv.shift = shift;
    dv.add = 0;
  }
  return dv;
}

extern "C" uint32_t cuttHipDivide(uint32_t n, cuttHipDivisor dv) {
  const uint32_t hi = (uint32_t)(((uint64_t)n * dv.mul) >> 32);
  return (hi + n * dv.add) >> dv.shift;
}

extern "C" int cuttHipFinishMbar(cuttHipMbar* mb) {
  if (!mb || mb->n < 0 || mb->n > CUTT_MAX_RANK) return -1;
  uint64_t below = 1;
  for (int k = 0; k < CUTT_MAX_RANK; k++) {
    cuttHipMbarDim& d = mb->d[k];
    if (k >= mb->n) {
      d.belowMul = d.extentMul = d.ctl = 0;  // quotients 0: no contribution
      continue;
    }
    if (d.extent == 0 || below * d.extent >= (1ull << 31)) return -1;
    const cuttHipDivisor b = cuttHipMakeDivisor((uint32_t)below), e = cuttHipMakeDivisor(d.extent);
    d.belowMul = b.mul;
    d.extentMul = e.mul;
    d.ctl = b.shift | (e.shift << 8) | (b.add << 16) | (e.add << 17);
    below *= d.extent;
  }
  return 0;
}

static int finishTileDigits(cuttHipTileDigits* dg, const cuttHipMbar* mb);

extern "C" int cuttHipFinishTileDigits(cuttHipTileDigits* dg, const cuttHipMbar* mb) {
  if (!dg || !mb) return -1;
  finishTileDigits(dg, mb);
  if (!dg->lanes) {  // not decodable in one step: no half-filled table
    dg->total = 0;
    for (int i = 0; i < CUTT_MAX_TILE_DIGITS; i++) dg->lane[i] = cuttHipDigitLane{0u, 0u, 0u, 1u, 0u, 0u, 0u, 0u};
  }
  return 0;
}

static int finishTileDigits(cuttHipTileDigits* dg, const cuttHipMbar* mb) {
  dg->lanes = 0;
  dg->total = 0;
  for (int i = 0; i < CUTT_MAX_TILE_DIGITS; i++) dg->lane[i] = cuttHipDigitLane{0u, 0u, 0u, 1u, 0u, 0u, 0u, 0u};
  if (dg->n < 1 || dg->n > CUTT_MAX_TILE_DIGITS || mb->n < 0 || mb->n > CUTT_MAX_RANK) return 0;
  uint64_t below = 1, mbarDigits = 1, volMbar = 1;
  for (int k = 0; k < mb->n; k++) volMbar *= mb->d[k].extent;
  for (int i = 0; i < dg->n; i++) {
    const cuttHipTileDigit& d = dg->d[i];
    cuttHipDigitLane& l = dg->lane[i];
    if (d.radix < 1 || d.which > 2 || below * d.radix >= (1ull << 31)) return 0;
    const cuttHipDivisor b = cuttHipMakeDivisor((uint32_t)below), e = cuttHipMakeDivisor(d.radix);
    l.belowMul = b.mul;
    l.radixMul = e.mul;
    l.ctl = b.shift | (e.shift << 8) | (b.add << 16) | (e.add << 17);
    l.radix = d.radix;
    if (d.which == 0) l.stepM = d.weight;
    if (d.which == 1) l.stepK = d.weight;
    if (d.which == 2 && d.radix > 1) {
      // the Mbar rank the digit counts in; it must not reach into the next one
      uint64_t rankBelow = 1;
      int k = 0;
      for (; k < mb->n; rankBelow *= mb->d[k].extent, k++)
        if ((uint64_t)d.weight >= rankBelow && (uint64_t)d.weight < rankBelow * mb->d[k].extent) break;
      if (k == mb->n || (uint64_t)d.weight % rankBelow != 0) return 0;
      const uint64_t u = (uint64_t)d.weight / rankBelow;
      if ((uint64_t)mb->d[k].extent % (u * d.radix) != 0) return 0;
      mbarDigits *= d.radix;
      if (u * mb->d[k].strideIn > 0xffffffffull || u * mb->d[k].strideOut > 0xffffffffull) return 0;
      l.strideIn = (uint32_t)(u * mb->d[k].strideIn);
      l.strideOut = (uint32_t)(u * mb->d[k].strideOut);
    }
    below *= d.radix;
  }
  // (no Mbar position beyond the last one: the kernels do not rebuild the position to check it)
  if (mbarDigits != volMbar) return 0;
  dg->total = (uint32_t)below;
  dg->lanes = 1;
  return 0;
}

extern "C" long long cuttHipPackedItemNumbers(const cuttHipPackedArgs* a) {
  const unsigned long long slabs = (unsigned long long)a->split[0].numSplit * (unsigned long long)a->split[1].numSplit;
  unsigned long long n = (unsigned long long)a->volMbar * slabs;
  if (a->itemOrder == 1) {
    const unsigned long long ipb = (unsigned long long)a->itemsPerBlock;
    n = (((unsigned long long)a->volMbar + ipb - 1) / ipb) * slabs * ipb;
  }
  return n > 0x7fffffffull ? -1 : (long long)n;
}

extern "C" int cuttHipDecodeItem(const cuttHipPackedArgs* a, uint32_t w, uint32_t* m, uint32_t* s0, uint32_t* s1, int* cls) {
  const uint32_t ns0 = (uint32_t)a->split[0].numSplit, ns1 = (uint32_t)a->split[1].numSplit;
  uint32_t slab = w, mi = 0, ipb = 1;
  if (a->itemOrder == 1) {
    ipb = (uint32_t)a->itemsPerBlock;
    slab = w / ipb;
    mi = w - slab * ipb;
  }
  const uint32_t t = cuttHipDivide(slab, a->split[0].div);
  *s0 = slab - t * ns0;
  const uint32_t mb = cuttHipDivide(t, a->split[1].div);
  *s1 = t - mb * ns1;
  *m = mb * ipb + mi;
  *cls = (*s0 < (uint32_t)a->split[0].slabRem ? 1 : 0) + (*s1 < (uint32_t)a->split[1].slabRem ? 2 : 0);
  return *m < (uint32_t)a->volMbar;
}

extern "C" size_t cuttHipPackedLdsBytes(const cuttHipPackedArgs* a) {
  const size_t b = (size_t)a->ldsElems * a->elemSize;
  return (b + 15) & ~(size_t)15;
}

// Registers per lane of packedKernel<T, E, *, WIDE> as compiled for gfx950 (the cache policy does
// not change the count).  Rows: E = 1, 2, 4, 8, 16.
extern "C" int cuttHipPackedRegsPerLane(int elemSize, int elemsPerThread, int wideOffsets) {
  static const int narrow4[5] = {15, 23, 38, 68, 124}, wide4[5] = {17, 27, 40, 72, 128};
  static const int narrow8[5] = {15, 25, 43, 73, 0}, wide8[5] = {18, 28, 48, 88, 0};
  int row = 0;
  while (row < 5 && (1 << row) != elemsPerThread) row++;
  if (row == 5 || (elemSize != 4 && elemSize != 8)) return 0;
  return elemSize == 4 ? (wideOffsets ? wide4 : narrow4)[row] : (wideOffsets ? wide8 : narrow8)[row];
}
