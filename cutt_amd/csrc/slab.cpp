/*
 * slab.cpp - cutting a tensor into pieces that one launch can address (see slab.h).
 */
#include "slab.h"

#include <algorithm>
#include <cstdlib>

namespace cutt {

int64_t slabSpanLimit() {
  if (const char* e = std::getenv("CUTT_SPAN_LIMIT")) {
    const long long v = std::atoll(e);
    if (v >= 2 && v < 0xffffffffll) return v;
  }
  return 0xffffffffll;
}

bool slabNeeded(int rank, const int* dim, int64_t spanLimit) {
  // a dense tensor spans its volume on both sides
  int64_t vol = 1;
  for (int r = 0; r < rank; r++) {
    vol *= dim[r];
    if (vol > spanLimit) return true;
  }
  return false;
}

bool slabDecompose(int rank, const int* dim, const int* perm, int elemSize, int64_t spanLimit,
                   SlabDecomposition& out) {
  out.shapes.clear();
  out.pieces.clear();
  std::vector<int64_t> sIn(rank), sOut(rank);
  int64_t c = 1;
  for (int r = 0; r < rank; r++) { sIn[r] = c; c *= dim[r]; }
  c = 1;
  for (int j = 0; j < rank; j++) { sOut[perm[j]] = c; c *= dim[perm[j]]; }

  // Extent of every rank inside one piece.  Per side, from the slowest rank down: a rank whose
  // faster ranks alone exceed the limit is fixed to one index; the first rank that fits partly is
  // cut to the largest extent that fits, and the span is within the limit.
  // The rank that leads a side (stride 1 there) is passed over as long as the other ranks can bring
  // the span down: a piece in which that rank had a single entry left would have no contiguous rows
  // on that side - (3, 40000, 40000) -> (40000, 40000, 3) cuts ranks 1 and 2 into four equal
  // pieces, where cutting rank 0 into 2 + 1 left a piece that no kernel can address.
  std::vector<int64_t> e(dim, dim + rank);
  const int leadIn = 0, leadOut = perm[0];
  auto spanOf = [&](const std::vector<int64_t>& stride) {
    int64_t span = 1;
    for (int r = 0; r < rank; r++) span += (e[r] - 1) * stride[r];
    return span;
  };
  // Three attempts per side: without either leading rank; without the other side's leading rank (this
  // side's own leading rank has stride 1 here, its pieces keep whole rows); with every rank.
  auto shrink = [&](const std::vector<int64_t>& stride, auto rankAt, int ownLead, int otherLead) {
    for (int pass = 0; pass < 3; pass++) {
      const std::vector<int64_t> before = e;
      for (int j = rank - 1; j >= 0; j--) {
        const int64_t span = spanOf(stride);
        if (span <= spanLimit) return;
        const int r = rankAt(j);
        if ((pass == 0 && r == ownLead) || (pass <= 1 && r == otherLead)) continue;
        const int64_t rest = span - (e[r] - 1) * stride[r];
        e[r] = rest > spanLimit ? 1 : std::min<int64_t>(e[r], (spanLimit - rest) / stride[r] + 1);
      }
      if (spanOf(stride) <= spanLimit) return;
      if (pass < 2) e = before;
    }
  };
  shrink(sIn, [&](int j) { return j; }, leadIn, leadOut);
  shrink(sOut, [&](int j) { return perm[j]; }, leadOut, leadIn);

  // Pieces per rank, evened out so that the last piece is not a sliver.
  std::vector<int64_t> count(rank), last(rank);
  int64_t numPieces = 1;
  std::vector<int> odd;  // cut ranks whose last piece is shorter
  for (int r = 0; r < rank; r++) {
    count[r] = (dim[r] + e[r] - 1) / e[r];
    e[r] = (dim[r] + count[r] - 1) / count[r];
    count[r] = (dim[r] + e[r] - 1) / e[r];
    last[r] = dim[r] - (count[r] - 1) * e[r];
    if (last[r] != e[r]) odd.push_back(r);
    numPieces *= count[r];
    if (numPieces > (1ll << 20)) return false;
  }
  if (odd.size() > 2) return false;  // more shapes of piece than a plan holds

  // One shape per combination of "last piece or not" of the ranks in `odd`.
  const int numShapes = 1 << odd.size();
  std::vector<int> shapeOf(numShapes, -1);
  auto extentIn = [&](int r, int mask) {
    for (size_t i = 0; i < odd.size(); i++)
      if (odd[i] == r && (mask >> i & 1)) return last[r];
    return e[r];
  };
  auto makeShape = [&](int mask) -> bool {
    std::vector<int> keep;  // ranks with more than one entry, in input order
    for (int r = 0; r < rank; r++)
      if (extentIn(r, mask) > 1) keep.push_back(r);
    std::vector<int> sdim, sperm;
    std::vector<int64_t> ssIn, ssOut;
    if (keep.empty()) {  // a single element: a one-entry rank keeps the problem well-formed
      sdim = {1}; sperm = {0}; ssIn = {1}; ssOut = {1};
    } else {
      for (int r : keep) {
        sdim.push_back((int)extentIn(r, mask));
        ssIn.push_back(sIn[r]);
        ssOut.push_back(sOut[r]);
      }
      for (int j = 0; j < rank; j++) {
        const auto it = std::find(keep.begin(), keep.end(), perm[j]);
        if (it != keep.end()) sperm.push_back((int)(it - keep.begin()));
      }
    }
    Problem p;
    if (!p.setStrided((int)sdim.size(), sdim.data(), sperm.data(), elemSize, ssIn.data(), ssOut.data())) return false;
    shapeOf[mask] = (int)out.shapes.size();
    out.shapes.push_back(std::move(p));
    return true;
  };

  // Enumerate the pieces (rank 0 fastest).
  std::vector<int64_t> idx(rank, 0);
  out.pieces.reserve((size_t)numPieces);
  for (int64_t n = 0; n < numPieces; n++) {
    int mask = 0;
    SlabPiece piece{0, 0, 0};
    for (int r = 0; r < rank; r++) {
      piece.baseIn += idx[r] * e[r] * sIn[r];
      piece.baseOut += idx[r] * e[r] * sOut[r];
    }
    for (size_t i = 0; i < odd.size(); i++)
      if (idx[odd[i]] == count[odd[i]] - 1) mask |= 1 << i;
    if (shapeOf[mask] < 0 && !makeShape(mask)) return false;
    piece.shape = shapeOf[mask];
    out.pieces.push_back(piece);
    for (int r = 0; r < rank; r++) {
      if (++idx[r] < count[r]) break;
      idx[r] = 0;
    }
  }
  return true;
}

}  // namespace cutt
