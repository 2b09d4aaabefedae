/*
 * slab.h - tensors beyond what one launch can address.
 *
 * The kernels keep positions as unsigned 32-bit element offsets from the base pointers they are
 * given.  A tensor whose input or output spans 2^32 elements and more is therefore transposed
 * piece by piece: the slowest ranks of each side are cut (or fixed to one index at a time) until a
 * piece spans less than the limit on both sides.  A piece is a transpose problem of its own with
 * the large tensor's strides (Problem::setStrided) and a base offset on each side; pieces of equal
 * shape share one plan.  The reference has no counterpart (its int volumes end at 2^31 - 1 elements).
 */
#ifndef CUTT_SLAB_H
#define CUTT_SLAB_H

#include <cstdint>
#include <vector>

#include "plan.h"

namespace cutt {

struct SlabPiece {
  int shape;                 // index into SlabDecomposition::shapes
  int64_t baseIn, baseOut;   // element offsets of the piece in the large tensors
};

struct SlabDecomposition {
  std::vector<Problem> shapes;    // at most four: a cut rank may leave a shorter last piece, on each side
  std::vector<SlabPiece> pieces;  // every element of the large tensor belongs to exactly one piece
};

// Largest element span of one piece: 2^32 - 1 unless CUTT_SPAN_LIMIT (tests) says less.
int64_t slabSpanLimit();

// True if a tensor of these (fused) extents needs cutting under `spanLimit`.
bool slabNeeded(int rank, const int* dim, int64_t spanLimit);

// Cuts the tensor (rank-fused already: ranks that stay adjacent must not be fused afterwards).
// False if no decomposition exists in which the leading rank of each side keeps stride 1 (a rank of
// 2^31 and more entries next to a tiny one), or if it would take more than 2^20 pieces.
bool slabDecompose(int rank, const int* dim, const int* perm, int elemSize, int64_t spanLimit,
                   SlabDecomposition& out);

}  // namespace cutt

#endif  // CUTT_SLAB_H
