/*
 * packed_items.h - device code shared by the packed transpose kernel and the kernel that replays its
 * address stream: which work items a workgroup handles (cuttHipPackedArgs.itemOrder) and where an
 * item's staged block lies in the two tensors.
 */
#ifndef CUTT_PACKED_ITEMS_H
#define CUTT_PACKED_ITEMS_H

#include <hip/hip_runtime.h>

#include "hip_layer.h"
#include "mbar_decode.h"
#include "tile_order.h"

namespace cutt {

// The work items of one workgroup: the numbers wBase + i * wStride, i < count.
struct PackedItems {
  uint32_t lb;       // logical index of the workgroup (XCD-aware renumbering applied)
  uint32_t wBase, wStride, count;
  bool byMbar;       // item order 1: the workgroup keeps its slabs and walks Mbar positions
};

__device__ __forceinline__ PackedItems packedItems(const cuttHipPackedArgs& a) {
  PackedItems it;
  const uint32_t ns0 = a.split[0].numSplit, ns1 = a.split[1].numSplit;
  const uint32_t ipb = (uint32_t)a.itemsPerBlock;
  it.byMbar = a.itemOrder == 1;
  const uint32_t totalItems = it.byMbar ? (((uint32_t)a.volMbar + ipb - 1) / ipb) * ns0 * ns1 * ipb
                                        : (uint32_t)a.volMbar * ns0 * ns1;
  // XCD-aware numbering: XCD x (= blockIdx.x % 8) walks its own contiguous chunk of the work
  // items, so that neighbouring slabs and Mbar positions share an L2.
  it.lb = blockIdx.x;
  if (a.xcdChunk) it.lb = (blockIdx.x % kNumXcd) * (uint32_t)a.xcdChunk + blockIdx.x / kNumXcd;
  // Orders 0 and 1: ipb consecutive numbers.  Order 2: the workgroups of one XCD take the numbers
  // of their chunk in turn, so that the items in flight at one time are neighbours and a
  // workgroup's next item lies a whole round ahead.
  it.wBase = it.lb * ipb;
  it.wStride = 1;
  it.count = it.wBase < totalItems ? min(ipb, totalItems - it.wBase) : 0;
  if (a.itemOrder == 2) {
    const uint32_t chunkBlocks = a.xcdChunk ? (uint32_t)a.xcdChunk : gridDim.x;
    const uint32_t x = it.lb / chunkBlocks;
    const uint32_t chunkStart = x * chunkBlocks * ipb;
    const uint32_t chunkEnd = min(chunkStart + chunkBlocks * ipb, totalItems);
    it.wBase = chunkStart + (it.lb - x * chunkBlocks);
    it.wStride = chunkBlocks;
    it.count = it.wBase < chunkEnd ? (chunkEnd - it.wBase + it.wStride - 1) / it.wStride : 0;
  }
  if (it.byMbar && it.count) {
    // the numbers of this workgroup whose Mbar position lies beyond the rank's end are empty
    const cuttHipDivisor d0 = a.split[0].div, d1 = a.split[1].div;
    const uint32_t mFirst = fastDivide(fastDivide(it.lb, d0.mul, d0.shift, d0.add), d1.mul, d1.shift, d1.add) * ipb;
    it.count = mFirst >= (uint32_t)a.volMbar ? 0 : min(it.count, (uint32_t)a.volMbar - mFirst);
  }
  return it;
}

// The workgroup's i-th item -> slab class and the item's base offsets (all wave-uniform).
__device__ __forceinline__ void packedLocate(const cuttHipPackedArgs& a, const PackedItems& it, const MbarLane& mbarLane,
                                             uint32_t i, int& cls, uint32_t& offIn, uint32_t& offOut) {
  const cuttHipDivisor div0 = a.split[0].div, div1 = a.split[1].div;
  const uint32_t ns0 = a.split[0].numSplit, ns1 = a.split[1].numSplit;
  const uint32_t rem0 = a.split[0].slabRem, rem1 = a.split[1].slabRem;
  const uint32_t slab = it.byMbar ? it.lb : it.wBase + i * it.wStride;
  const uint32_t t = fastDivide(slab, div0.mul, div0.shift, div0.add);
  const uint32_t s0 = slab - t * ns0;
  uint32_t m = fastDivide(t, div1.mul, div1.shift, div1.add);
  const uint32_t s1 = t - m * ns1;
  if (it.byMbar) m = m * (uint32_t)a.itemsPerBlock + i;
  cls = (s0 < rem0 ? 1 : 0) + (s1 < rem1 ? 2 : 0);
  const uint32_t p0 = s0 * (uint32_t)a.split[0].slabFloor + min(s0, rem0);
  const uint32_t p1 = s1 * (uint32_t)a.split[1].slabFloor + min(s1, rem1);
  mbarOffsets(mbarLane, m, offIn, offOut);
  offIn += p0 * a.split[0].strideIn + p1 * a.split[1].strideIn;
  offOut += p0 * a.split[0].strideOut + p1 * a.split[1].strideOut;
}

// Element index p of a staged block -> offset inside the block's input / output footprint, from the
// class's run tables (one offset per contiguous run).
__device__ __forceinline__ uint32_t packedInElem(const cuttHipPackedClass& k, uint32_t p) {
  const uint32_t ri = fastDivide(p, k.inDiv.mul, k.inDiv.shift, k.inDiv.add);
  // uniform base + 32-bit lane offset (the tables are far smaller than 4 GB)
  const uint32_t rowI = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const unsigned char*>(k.rowIn) + ri * 4u);
  return rowI + (p - ri * (uint32_t)k.inCont);
}

__device__ __forceinline__ uint32_t packedOutElem(const cuttHipPackedClass& k, uint32_t p) {
  const uint32_t ro = fastDivide(p, k.outDiv.mul, k.outDiv.shift, k.outDiv.add);
  const uint32_t rowO = *reinterpret_cast<const uint32_t*>(reinterpret_cast<const unsigned char*>(k.rowOut) + ro * 4u);
  return rowO + (p - ro * (uint32_t)k.outCont);
}

}  // namespace cutt

#endif  // CUTT_PACKED_ITEMS_H
