/*
 * tile_order.h - device code shared by the tiled transpose kernels and the kernels that replay
 * their address streams: the tile geometry and the mapping from a workgroup's index to the tile
 * and the Mbar position it handles.
 */
#ifndef CUTT_TILE_ORDER_H
#define CUTT_TILE_ORDER_H

#include <hip/hip_runtime.h>

#include "hip_layer.h"

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
constexpr uint32_t kNumXcd = 8;

struct TileOrder {
  int order;
  uint32_t xcdChunk, superM, superK;
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

}  // namespace cutt

#endif  // CUTT_TILE_ORDER_H
