/*
 * tile_order.h - device code shared by the tiled transpose kernels and the kernels that replay
 * their address streams: the tile geometry and the mapping from a workgroup's index to the tile
 * and the Mbar position it handles.
 */
#ifndef CUTT_TILE_ORDER_H
#define CUTT_TILE_ORDER_H

#include <hip/hip_runtime.h>

#include "hip_layer.h"
#include "mbar_decode.h"

namespace cutt {

constexpr int kTile = 64;             // tile edge in elements
constexpr int kTileThreads = 256;     // 4 wavefronts
constexpr int kTileRows = kTile * kTile / kTileThreads;  // rows per lane: 16
constexpr int kGroupRows = 4;                            // rows per lane in one skippable group
constexpr int kRowGroups = kTileRows / kGroupRows;       // 4 groups of 16 tile rows each
constexpr int kWaves = kTileThreads / 64;

// Workgroup index -> (tile along Mm, tile along Mk, Mbar position).  Returns false for the
// padding workgroups of order 3.
//
// The chip has 8 XCDs with private L2s and hands workgroup b to XCD b % 8, so neighbouring
// tiles - which share the 128-byte lines at their unaligned edges - would otherwise always land
// in different L2s.  With xcdChunk != 0, XCD x walks its own contiguous chunk of the logical
// sequence.  Orders 0-2 number the logical sequence with the Mbar position, the tile along Mm or
// the tile along Mk running fastest; orders 3 and 4 visit the tiles in superM x superK super-tiles, so
// that both the read neighbours (along Mm) and the write neighbours (along Mk) of a tile are
// resident in the same L2 at about the same time.  Order 5 is order 3 with the Mbar position running
// between the super-tiles: the runs of consecutive Mbar positions, which are neighbours in memory
// when the fastest Mbar rank follows Mk in the output (or Mm in the input), then meet in the L2 too.
// Order 6 is order 5 with another numbering of the super-tiles: along Mk first, and the super-tile row at
// index mi along Mm starts at column mi (mod the columns).  XCDs that own different rows then work on
// different columns at any one time, and with small patches their reads and their writes both spread over
// the address space (measured on C2: 2 x 2 patches 5.3 TB/s in order 5, 6.15 TB/s in order 6; which shapes
// gain is not predictable from the strides, so only the measuring planner uses it).
// Order 7 reads the logical index as a mixed-radix number whose digits are dealt out to the three
// coordinates (cuttHipTileDigits): any nesting of patches, strips and Mbar runs can be written that way.
constexpr uint32_t kNumXcd = 8;

struct TileOrder {
  int order;
  uint32_t xcdChunk, superM, superK;
  const cuttHipTileDigits* digits;  // order 7 (points into the kernel arguments)
};

__device__ __forceinline__ bool decodeTile(uint32_t bid, const TileOrder o, uint32_t tilesM,
                                           uint32_t tilesK, uint32_t volMbar, uint32_t& tm,
                                           uint32_t& tk, uint32_t& m) {
  const uint32_t l = o.xcdChunk ? (bid % kNumXcd) * o.xcdChunk + bid / kNumXcd : bid;
  if (o.order == 0) {
    const uint32_t t = l / volMbar;
    m = l - t * volMbar;
    tk = t / tilesM;
    tm = t - tk * tilesM;
    return tk < tilesK;
  } else if (o.order == 1) {
    const uint32_t t = l / tilesM;
    tm = l - t * tilesM;
    m = t / tilesK;
    tk = t - m * tilesK;
    return m < volMbar;
  } else if (o.order == 2) {
    const uint32_t t = l / tilesK;
    tk = l - t * tilesK;
    m = t / tilesM;
    tm = t - m * tilesM;
    return m < volMbar;
  } else if (o.order == 7) {
    const cuttHipTileDigits& dg = *o.digits;
    uint32_t c0 = 0, c1 = 0, c2 = 0, rest = l;
    for (int i = 0; i < dg.n; i++) {
      const cuttHipTileDigit d = dg.d[i];
      const uint32_t q = fastDivide(rest, d.div.mul, d.div.shift, d.div.add);
      // the slowest digit takes what is left (beyond its radix on the padding workgroups)
      const uint32_t v = (i + 1 < dg.n ? rest - q * d.radix : rest) * d.weight;
      rest = q;
      if (d.which == 0) c0 += v;
      else if (d.which == 1) c1 += v;
      else c2 += v;
    }
    tm = c0; tk = c1; m = c2;
    return tm < tilesM && tk < tilesK && m < volMbar;
  }
  const uint32_t nSuperM = (tilesM + o.superM - 1) / o.superM, nSuperK = (tilesK + o.superK - 1) / o.superK;
  const uint32_t per = o.superM * o.superK;
  const uint32_t w = l % per;
  const uint32_t t = l / per;
  uint32_t st;
  if (o.order >= 5) {  // like 3, but a super-tile is visited for every Mbar position in turn
    st = t / volMbar;
    m = t - st * volMbar;
    if (st >= nSuperM * nSuperK) return false;
  } else {
    st = t % (nSuperM * nSuperK);
    m = t / (nSuperM * nSuperK);
  }
  if (o.order == 6) {  // super-tiles along Mk first, row mi rotated by mi columns
    const uint32_t mi = st / nSuperK, ki = (st - mi * nSuperK + mi) % nSuperK;
    tm = mi * o.superM + (w % o.superM);
    tk = ki * o.superK + (w / o.superM);
  } else if (o.order != 4) {  // inside a super-tile the tiles along Mm run fastest
    tm = (st % nSuperM) * o.superM + (w % o.superM);
    tk = (st / nSuperM) * o.superK + (w / o.superM);
  } else {             // order 4: the tiles along Mk run fastest, super-tiles advance along Mk first
    tk = (st % nSuperK) * o.superK + (w % o.superK);
    tm = (st / nSuperK) * o.superM + (w / o.superK);
  }
  return m < volMbar && tm < tilesM && tk < tilesK;
}

// Workgroup index -> tile coordinates and the offsets of its Mbar position (all wave-uniform); false for
// a padding workgroup.  With a digit list that the host could turn into lanes (cuttHipFinishTileDigits)
// lane i of every row of 16 lanes takes digit i - two multiply-high divisions give its value - and four row
// sums add up what the digits contribute; nothing is read digit by digit.  Otherwise decodeTile and the
// Mbar table.
template <typename Args>
__device__ __forceinline__ bool locateTile(const Args& a, uint32_t& tm, uint32_t& tk, uint32_t& offIn, uint32_t& offOut) {
  if (a.order == 7 && a.digits.lanes) {
    const uint32_t l = a.xcdChunk ? (blockIdx.x % kNumXcd) * a.xcdChunk + blockIdx.x / kNumXcd : blockIdx.x;
    if (l >= a.digits.total) return false;
    static_assert(CUTT_MAX_TILE_DIGITS == 16, "one DPP row of 16 lanes holds the digits");
    const cuttHipDigitLane d = a.digits.lane[threadIdx.x & 15];  // (entries beyond the list contribute 0)
    const uint32_t q = fastDivide(l, d.belowMul, d.ctl & 0xff, (d.ctl >> 16) & 1);
    const uint32_t q2 = fastDivide(q, d.radixMul, (d.ctl >> 8) & 0xff, (d.ctl >> 17) & 1);
    const uint32_t v = q - q2 * d.radix;
    tm = (uint32_t)__builtin_amdgcn_readfirstlane((int)rowSum(v * d.stepM));
    tk = (uint32_t)__builtin_amdgcn_readfirstlane((int)rowSum(v * d.stepK));
    offIn = (uint32_t)__builtin_amdgcn_readfirstlane((int)rowSum(v * d.strideIn));
    offOut = (uint32_t)__builtin_amdgcn_readfirstlane((int)rowSum(v * d.strideOut));
    return tm < (uint32_t)a.tilesM && tk < (uint32_t)a.tilesK;
  }
  uint32_t m;
  if (!decodeTile(blockIdx.x, TileOrder{a.order, a.xcdChunk, a.superM, a.superK, &a.digits}, a.tilesM, a.tilesK, a.volMbar, tm, tk, m)) return false;
  mbarOffsets(loadMbarLane(a.mbar, threadIdx.x & 63), m, offIn, offOut);
  return true;
}

// Offset of row `i` of a tile axis that runs over the fused ranks of `rr` (rr.n >= 1), per lane.
__device__ __forceinline__ uint32_t rowOffset(const cuttHipRowRadix& rr, uint32_t i) {
  uint32_t off = 0;
  for (int k = 0; k + 1 < rr.n; k++) {
    const uint32_t q = fastDivide(i, rr.div[k].mul, rr.div[k].shift, rr.div[k].add);
    off += (i - q * rr.extent[k]) * rr.stride[k];
    i = q;
  }
  return off + i * rr.stride[rr.n - 1];
}

// The offsets of the 64 rows of a tile that starts at row `first` of an axis with `count` rows, one
// row per lane (rows beyond the axis repeat the last one); `stride` is used when the axis is a single rank.
__device__ __forceinline__ uint32_t tileRowOffsets(const cuttHipRowRadix& rr, uint32_t stride, uint32_t first,
                                                   uint32_t count, uint32_t lane) {
  const uint32_t i = min(first + lane, count - 1);
  return rr.n > 0 ? rowOffset(rr, i) : i * stride;
}

// What a lane of a Tiled workgroup needs to address the rows of its tile; shared by the transpose
// kernel and the kernel that replays its address stream.
struct TileLanes {
  uint32_t m0, k0;            // first element of the tile along Mm / Mk
  uint32_t wM, wK;            // last valid column / row inside the tile (edge tiles are narrower)
  uint32_t groupsM, groupsK;  // groups of 16 rows that hold valid rows, per side
  uint32_t cx, ck;            // the lane's (clamped) position along Mm when reading, along Mk when writing
  uint32_t rdBase, wrBase;    // element offset of the lane's column in row 0 of the tile's axis origin
  uint32_t rowK, rowM, waveU; // FUSED: row offsets held one per lane, and the wave index as a scalar
};

template <bool FUSED>
__device__ __forceinline__ TileLanes tileLanes(const cuttHipTiledArgs& a, uint32_t tm, uint32_t tk, uint32_t offIn,
                                               uint32_t offOut, uint32_t lane, uint32_t wave) {
  TileLanes t;
  t.m0 = tm * kTile;
  t.k0 = tk * kTile;
  // Edge tiles are handled without branches: indices are clamped to the last valid row / column,
  // so out-of-range lanes repeat the access of the edge element (same address, same value).  That
  // keeps the loop bodies straight-line code, and all 16 loads of a lane go out back to back.
  t.wM = min((uint32_t)kTile, (uint32_t)a.volMm - t.m0) - 1;
  t.wK = min((uint32_t)kTile, (uint32_t)a.volMk - t.k0) - 1;
  // The 16 rows of a lane come in kRowGroups groups of 4; group g covers tile rows 16g..16g+15
  // over the four waves.  An edge tile skips the groups that lie entirely beyond its valid part
  // (a test that is uniform over the workgroup), so that a thin edge costs a quarter of a tile's
  // instructions, not all of them; inside a group the clamping above still applies.
  t.groupsK = (t.wK >> 4) + 1;
  t.groupsM = (t.wM >> 4) + 1;
  t.cx = min(lane, t.wM);
  t.ck = min(lane, t.wK);
  t.rdBase = offIn + t.m0 + t.cx;
  t.wrBase = offOut + t.k0 + t.ck;
  t.rowK = t.rowM = t.waveU = 0;
  if constexpr (FUSED) {
    // lane l holds the input offset of row k0 + l along Mk and the output offset of row m0 + l along
    // Mm; the row a wave asks for is wave-uniform
    t.rowK = tileRowOffsets(a.rowsK, a.strideInK, t.k0, (uint32_t)a.volMk, lane);
    t.rowM = tileRowOffsets(a.rowsM, a.strideOutM, t.m0, (uint32_t)a.volMm, lane);
    t.waveU = (uint32_t)__builtin_amdgcn_readfirstlane((int)wave);
  }
  return t;
}

// Element offset of the lane's j-th load (row wave + 4 j of the tile, clamped) / store.
template <bool FUSED>
__device__ __forceinline__ uint32_t tileReadElem(const TileLanes& t, const cuttHipTiledArgs& a, uint32_t wave, int j) {
  if constexpr (FUSED) {
    const uint32_t r = min(t.waveU + kWaves * j, t.wK);
    return t.rdBase + (uint32_t)__builtin_amdgcn_readlane((int)t.rowK, (int)r);
  } else {
    const uint32_t r = min(wave + kWaves * j, t.wK);
    return t.rdBase + (t.k0 + r) * a.strideInK;
  }
}

template <bool FUSED>
__device__ __forceinline__ uint32_t tileWriteElem(const TileLanes& t, const cuttHipTiledArgs& a, uint32_t wave, int j) {
  if constexpr (FUSED) {
    const uint32_t r = min(t.waveU + kWaves * j, t.wM);
    return t.wrBase + (uint32_t)__builtin_amdgcn_readlane((int)t.rowM, (int)r);
  } else {
    const uint32_t r = min(wave + kWaves * j, t.wM);
    return t.wrBase + (t.m0 + r) * a.strideOutM;
  }
}

}  // namespace cutt

#endif  // CUTT_TILE_ORDER_H
