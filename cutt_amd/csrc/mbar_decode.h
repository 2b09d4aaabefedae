/*
 * mbar_decode.h - device code that turns an Mbar position (the linear index over
 * the ranks a workgroup does not stage) into input and output offsets.
 *
 * Lane k of a wavefront owns Mbar rank k: it keeps that rank's division
 * constants and strides in registers, computes its index (m / below) % extent
 * with two multiply-high divisions, and the wavefront sums the 32 possible
 * contributions with four DPP adds per row of 16 lanes.  The cost does not
 * grow with the number of ranks and nothing is loaded from memory per item.
 * The reference assigns ranks to lanes in the same way and reduces with warp
 * shuffles (src/cuttkernel.cu:60-73,161-175).
 */
#ifndef CUTT_MBAR_DECODE_H
#define CUTT_MBAR_DECODE_H

#include <hip/hip_runtime.h>

#include "hip_layer.h"

namespace cutt {

// n / d for n < 2^31 (constants from cuttHipMakeDivisor).
__device__ __forceinline__ uint32_t fastDivide(uint32_t n, uint32_t mul, uint32_t shift, uint32_t add) {
  return (__umulhi(n, mul) + n * add) >> shift;
}

// One lane's share of the Mbar table.
struct MbarLane {
  uint32_t belowMul, extentMul, ctl, extent, strideIn, strideOut;
};

// Lane `lane` (0..63) takes rank `lane`; lanes beyond the table contribute nothing.
__device__ __forceinline__ MbarLane loadMbarLane(const cuttHipMbar& mb, uint32_t lane) {
  const cuttHipMbarDim& d = mb.d[lane < (uint32_t)CUTT_MAX_RANK ? lane : 0];
  const bool live = lane < (uint32_t)mb.n;
  MbarLane l;
  l.belowMul = d.belowMul;
  l.extentMul = d.extentMul;
  l.ctl = d.ctl;
  l.extent = d.extent;
  l.strideIn = live ? d.strideIn : 0u;
  l.strideOut = live ? d.strideOut : 0u;
  return l;
}

// Sum over the 16 lanes of each DPP row; every lane of a row ends up with the row's sum.
__device__ __forceinline__ uint32_t rowSum(uint32_t v) {
  // lane ^ 1, lane ^ 2 inside quads, then the mirrored half-row and the mirrored row
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, false);   // quad_perm [1,0,3,2]
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, false);   // quad_perm [2,3,0,1]
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, false);  // row_half_mirror
  v += (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x140, 0xF, 0xF, false);  // row_mirror
  return v;
}

// Offsets of Mbar position m (wave-uniform); every lane returns the same values.
// CUTT_MAX_RANK is 32, so the live ranks sit in rows 0 and 1 of the wavefront.
__device__ __forceinline__ void mbarOffsets(const MbarLane& l, uint32_t m, uint32_t& offIn, uint32_t& offOut) {
  static_assert(CUTT_MAX_RANK == 32, "the row sums below cover lanes 0..31");
  const uint32_t q = fastDivide(m, l.belowMul, l.ctl & 0xff, (l.ctl >> 16) & 1);
  const uint32_t q2 = fastDivide(q, l.extentMul, (l.ctl >> 8) & 0xff, (l.ctl >> 17) & 1);
  const uint32_t idx = q - q2 * l.extent;
  const uint32_t si = rowSum(idx * l.strideIn);
  const uint32_t so = rowSum(idx * l.strideOut);
  offIn = (uint32_t)__builtin_amdgcn_readlane((int)si, 0) + (uint32_t)__builtin_amdgcn_readlane((int)si, 16);
  offOut = (uint32_t)__builtin_amdgcn_readlane((int)so, 0) + (uint32_t)__builtin_amdgcn_readlane((int)so, 16);
}

}  // namespace cutt

#endif  // CUTT_MBAR_DECODE_H
