/*
 * plan.cpp - host planner.  See plan.h.
 *
 * Behaviour follows the reference planner (rank fusing src/cuttplan.cpp:63-126,
 * index-set volumes :201-280, candidate enumeration :475-698, index tables
 * :817-1046, launch rules src/cuttkernel.cu:665-838); the geometry is derived
 * for gfx950: 64-lane wavefronts, 64x64 tiles, up to 160 KB of LDS per
 * workgroup, short-lived workgroups.
 */
#include "plan.h"

#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <sstream>

namespace cutt {

namespace {
constexpr int kTile = 64;
constexpr int kPadShift = 5;            // one LDS pad slot per 32 elements
constexpr int64_t kMaxLdsSlots = 65536; // the gather index is 16 bits wide
constexpr int64_t kNumXcd = 8;          // XCDs (private L2s); workgroup b runs on XCD b % 8

inline int64_t ceilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int roundUp64(int64_t v) { return (int)(ceilDiv(v, 64) * 64); }
inline int64_t paddedSlots(int64_t vol, int shift = kPadShift) { return vol ? (vol - 1) + ((vol - 1) >> shift) + 1 : 0; }
}  // namespace

const char* methodName(int method) {
  switch (method) {
    case kTrivial: return "Trivial";
    case kPacked: return "Packed";
    case kPackedSplit: return "PackedSplit";
    case kTiled: return "Tiled";
    case kTiledCopy: return "TiledCopy";
    default: return "Unknown";
  }
}

cuttHipDeviceProps defaultMI355XProps() {
  cuttHipDeviceProps p;
  std::memset(&p, 0, sizeof(p));
  p.cuCount = 256;
  p.waveSize = 64;
  p.maxThreadsPerBlock = 1024;
  p.maxThreadsPerCU = 2048;
  p.ldsPerBlock = 160 * 1024;
  p.ldsPerCU = 160 * 1024;
  p.clockKHz = 2400000;
  p.memClockKHz = 2000000;
  p.memBusWidthBits = 8192;
  p.l2Bytes = 4 * 1024 * 1024;
  p.maxGridX = 2147483647;
  p.infinityCacheBytes = (size_t)256 << 20;
  std::strncpy(p.arch, "gfx950", sizeof(p.arch) - 1);
  return p;
}

// Runtimes and devices differ in what they report; a zero or implausible field would turn the
// model's copy time into infinity (every candidate then ties) or size the grids for no CUs at all.
void sanitizeDeviceProps(cuttHipDeviceProps& p) {
  const cuttHipDeviceProps d = defaultMI355XProps();
  if (p.cuCount < 1 || p.cuCount > 4096) p.cuCount = d.cuCount;
  if (p.waveSize != 32 && p.waveSize != 64) p.waveSize = d.waveSize;
  if (p.maxThreadsPerBlock < 64 || p.maxThreadsPerBlock > 1024) p.maxThreadsPerBlock = d.maxThreadsPerBlock;
  if (p.maxThreadsPerCU < p.maxThreadsPerBlock) p.maxThreadsPerCU = d.maxThreadsPerCU;
  if (p.ldsPerBlock < 16 * 1024) p.ldsPerBlock = std::min<size_t>(d.ldsPerBlock, 64 * 1024);
  if (p.ldsPerCU < p.ldsPerBlock) p.ldsPerCU = p.ldsPerBlock;
  if (p.clockKHz < 100000) p.clockKHz = d.clockKHz;
  // the product of memory clock and bus width is what the model uses (bytes per second)
  if (p.memClockKHz < 100000 || p.memBusWidthBits < 64) {
    p.memClockKHz = d.memClockKHz;
    p.memBusWidthBits = d.memBusWidthBits;
  }
  if (p.l2Bytes < 256 * 1024) p.l2Bytes = d.l2Bytes;
  if (p.maxGridX < 65535) p.maxGridX = d.maxGridX;
}

// ---------------------------------------------------------------------------
void Problem::set(int rank_, const int* dim_, const int* perm_, int elemSize_) {
  rank = rank_;
  elemSize = elemSize_;
  dim.assign(dim_, dim_ + rank);
  perm.assign(perm_, perm_ + rank);
  inv.assign(rank, 0);
  for (int j = 0; j < rank; j++) inv[perm[j]] = j;
  strideIn.assign(rank, 1);
  strideOut.assign(rank, 1);
  int64_t c = 1;
  for (int r = 0; r < rank; r++) {
    strideIn[r] = c;
    c *= dim[r];
  }
  volume = c;
  c = 1;
  for (int j = 0; j < rank; j++) {
    strideOut[perm[j]] = c;
    c *= dim[perm[j]];
  }
  gapIn.assign(rank, 0);
  gapOut.assign(rank, 0);
  dense = true;
  span = volume;
}

bool Problem::setStrided(int rank_, const int* dim_, const int* perm_, int elemSize_, const int64_t* strideIn_,
                         const int64_t* strideOut_) {
  set(rank_, dim_, perm_, elemSize_);
  strideIn.assign(strideIn_, strideIn_ + rank);
  strideOut.assign(strideOut_, strideOut_ + rank);
  if (rank < 1 || strideIn[0] != 1 || strideOut[perm[0]] != 1) return false;
  for (int r = 0; r + 1 < rank; r++) {
    gapIn[r] = strideIn[r + 1] != strideIn[r] * dim[r];
    const int a = perm[r], b = perm[r + 1];
    gapOut[a] = strideOut[b] != strideOut[a] * dim[a];
    if (gapIn[r] || gapOut[a]) dense = false;
  }
  int64_t spanIn = 1, spanOut = 1;
  for (int r = 0; r < rank; r++) {
    spanIn += (int64_t)(dim[r] - 1) * strideIn[r];
    spanOut += (int64_t)(dim[r] - 1) * strideOut[r];
  }
  span = std::max(spanIn, spanOut);
  return true;
}

void reduceRanks(int rank, const int* dim, const int* perm, std::vector<int>& redDim,
                 std::vector<int>& redPerm) {
  // Groups of output ranks whose input ranks are consecutive and increasing.
  std::vector<int> first, vol;
  for (int j = 0; j < rank; j++) {
    // (a fused extent must still fit an int; beyond that the ranks stay apart)
    if (j > 0 && perm[j] == perm[j - 1] + 1 && (int64_t)vol.back() * dim[perm[j]] < (1ll << 31)) {
      vol.back() *= dim[perm[j]];
    } else {
      first.push_back(perm[j]);
      vol.push_back(dim[perm[j]]);
    }
  }
  const int n = (int)first.size();
  // A group's new input rank = its position when groups are sorted by first input rank.
  std::vector<int> order(n);
  for (int g = 0; g < n; g++) order[g] = g;
  std::sort(order.begin(), order.end(), [&](int a, int b) { return first[a] < first[b]; });
  redDim.assign(n, 0);
  redPerm.assign(n, 0);
  for (int newRank = 0; newRank < n; newRank++) {
    const int g = order[newRank];
    redPerm[g] = newRank;
    redDim[newRank] = vol[g];
  }
}

// ---------------------------------------------------------------------------
void Split::update(int numMm_, int numMk_, const Problem& pb) {
  numMm = numMm_;
  numMk = numMk_;
  const int rank = pb.rank;
  inMmk.assign(rank, 0);
  volMm = volMk = volMmk = volMkBar = 1;
  sizeMmk = sizeMkBar = 0;
  for (int r = 0; r < numMm; r++) volMm *= pb.dim[r];
  for (int j = 0; j < numMk; j++) volMk *= pb.dim[pb.perm[j]];
  for (int r = 0; r < rank; r++) {
    const bool mm = r < numMm, mk = pb.inv[r] < numMk;
    if (mm || mk) {
      inMmk[r] = 1;
      sizeMmk++;
      volMmk *= pb.dim[r];
      if (!mm) {
        sizeMkBar++;
        volMkBar *= pb.dim[r];
      }
    }
  }
  sizeMbar = rank - sizeMmk;
  volMbar = pb.volume / volMmk;
  volMmkUnsplit = volMmk;
  for (int i = 0; i < 2; i++) {
    splitDim[i] = splitRank[i] >= 0 ? pb.dim[splitRank[i]] : 0;
    if (splitRank[i] >= 0) volMmkUnsplit /= splitDim[i];
  }
  volMmkInCont = 1;
  for (int r = 0; r < rank && inMmk[r]; r++) {
    const int slot = splitSlot(r);
    if (slot >= 0) {
      volMmkInCont *= slabMax(slot);
      break;
    }
    volMmkInCont *= pb.dim[r];
    if (pb.gapIn[r]) break;
  }
  volMmkOutCont = 1;
  for (int j = 0; j < rank && inMmk[pb.perm[j]]; j++) {
    const int r = pb.perm[j];
    const int slot = splitSlot(r);
    if (slot >= 0) {
      volMmkOutCont *= slabMax(slot);
      break;
    }
    volMmkOutCont *= pb.dim[r];
    if (pb.gapOut[r]) break;
  }
}

int64_t Split::volStaged() const {
  switch (method) {
    case kPacked: return volMmk;
    case kPackedSplit: return (int64_t)slabMax(0) * slabMax(1) * volMmkUnsplit;
    case kTiled: return kTile * kTile;
    default: return 0;
  }
}

// ---------------------------------------------------------------------------
Plan::Plan() {
  std::memset(&tiled, 0, sizeof(tiled));
  std::memset(&tcopy, 0, sizeof(tcopy));
  std::memset(&packed, 0, sizeof(packed));
  std::memset(&itemDigits, 0, sizeof(itemDigits));
}

Plan::~Plan() { release(); }

Plan::Plan(Plan&& o) noexcept { *this = std::move(o); }

Plan& Plan::operator=(Plan&& o) noexcept {
  if (this == &o) return *this;
  release();
  method = o.method;
  split = std::move(o.split);
  pb = std::move(o.pb);
  fromReduced = o.fromReduced;
  deviceID = o.deviceID;
  stream = o.stream;
  tiled = o.tiled;
  tcopy = o.tcopy;
  packed = o.packed;
  itemDigits = o.itemDigits;
  ldsBytes = o.ldsBytes;
  numBlocks = o.numBlocks;
  numThreads = o.numThreads;
  for (int c = 0; c < 4; c++) tab[c] = std::move(o.tab[c]);
  tablesBuilt = o.tablesBuilt;
  dTables = o.dTables;
  o.dTables = nullptr;
  launchable = o.launchable;
  o.launchable = false;
  model = o.model;
  return *this;
}

Plan Plan::clone() const {
  Plan q;
  q.method = method;
  q.split = split;
  q.pb = pb;
  q.fromReduced = fromReduced;
  q.deviceID = deviceID;
  q.stream = stream;
  q.tiled = tiled;
  q.tcopy = tcopy;
  q.packed = packed;
  q.itemDigits = itemDigits;
  for (int c = 0; c < 4; c++) {  // device tables stay with the original
    q.packed.cls[c].rowIn = nullptr;
    q.packed.cls[c].rowOut = nullptr;
    q.packed.cls[c].shIdx = nullptr;
  }
  q.ldsBytes = ldsBytes;
  q.numBlocks = numBlocks;
  q.numThreads = numThreads;
  for (int c = 0; c < 4; c++) q.tab[c] = tab[c];
  q.tablesBuilt = tablesBuilt;
  q.model = model;
  return q;
}

void Plan::release() {
  if (method == kPacked || method == kPackedSplit) launchable = false;
  if (dTables) {
    cuttHipFree(dTables);
    dTables = nullptr;
    for (int c = 0; c < 4; c++) {
      packed.cls[c].rowIn = nullptr;
      packed.cls[c].rowOut = nullptr;
      packed.cls[c].shIdx = nullptr;
    }
  }
}

namespace {

// Offsets of a mixed-radix enumeration: for every combination of indices over
// `dims` (first entry fastest) the sum of index*stride.
struct RadixDim {
  int extent;
  int64_t stride;
};

template <typename OutT>
void enumerateOffsets(const std::vector<RadixDim>& dims, int64_t count, std::vector<OutT>& out) {
  out.resize((size_t)count);
  std::vector<int> idx(dims.size(), 0);
  int64_t off = 0;
  for (int64_t i = 0; i < count; i++) {
    out[(size_t)i] = (OutT)off;
    for (size_t k = 0; k < dims.size(); k++) {
      off += dims[k].stride;
      if (++idx[k] < dims[k].extent) break;
      off -= (int64_t)dims[k].extent * dims[k].stride;
      idx[k] = 0;
    }
  }
}

// Mbar table.  The order of its ranks is the order in which consecutive workgroups walk the
// remaining index space: mbarOrder 0 = input order (consecutive workgroups read neighbouring
// memory), 1 = output order (they write neighbouring memory, so the partly written 128-byte
// lines at the ends of their runs meet in the same L2).
int64_t parseTileDigits(const std::string& text, int64_t tilesM, int64_t tilesK, int64_t volMbar, cuttHipTileDigits& dg);

bool fillMbar(const Problem& pb, const std::vector<char>& inMmk, int mbarOrder, cuttHipMbar& mb) {
  std::memset(&mb, 0, sizeof(mb));
  // Order of the Mbar ranks (first = fastest over consecutive work items):
  //   0 input order, 1 output order, 2 the first input rank outside Mmk, then output order.
  // Workgroups that run side by side on one XCD then touch neighbouring memory, and the lines at
  // the unaligned edges of their runs are shared in the L2: with 2 on the read side for the
  // nearest neighbour and on the write side for the next ones.
  std::vector<int> order;
  if (mbarOrder == 2)
    for (int r = 0; r < pb.rank; r++)
      if (!inMmk[r]) {
        order.push_back(r);
        break;
      }
  for (int i = 0; i < pb.rank; i++) {
    const int r = mbarOrder == 0 ? i : pb.perm[i];
    if (inMmk[r] || (!order.empty() && mbarOrder == 2 && r == order[0])) continue;
    order.push_back(r);
  }
  int n = 0;
  for (int r : order) {
    mb.d[n].extent = (uint32_t)pb.dim[r];
    mb.d[n].strideIn = (uint32_t)pb.strideIn[r];
    mb.d[n].strideOut = (uint32_t)pb.strideOut[r];
    n++;
  }
  mb.n = n;
  // Fails only when the extents multiply to 2^31 or more (a tensor of 2^31 elements and more with
  // a tiny Mmk); such a candidate is dropped.
  return cuttHipFinishMbar(&mb) == 0;
}

// Extent of rank r inside one staged block whose split ranks have the slab sizes slab[0..1].
inline int blockExtent(const Split& sp, const Problem& pb, int r, const int* slab) {
  const int slot = sp.splitSlot(r);
  return slot >= 0 ? slab[slot] : pb.dim[r];
}

// Geometry of one slab class: volume and contiguous run lengths.
void classGeometry(const Split& sp, const Problem& pb, const int* slab, int64_t& vol, int64_t& inCont,
                   int64_t& outCont) {
  int64_t v = 1, ic = 1, oc = 1;
  for (int r = 0; r < pb.rank; r++)
    if (sp.inMmk[r]) v *= blockExtent(sp, pb, r, slab);
  for (int r = 0; r < pb.rank && sp.inMmk[r]; r++) {
    ic *= blockExtent(sp, pb, r, slab);
    if (sp.splitSlot(r) >= 0 || pb.gapIn[r]) break;
  }
  for (int j = 0; j < pb.rank && sp.inMmk[pb.perm[j]]; j++) {
    const int r = pb.perm[j];
    oc *= blockExtent(sp, pb, r, slab);
    if (sp.splitSlot(r) >= 0 || pb.gapOut[r]) break;
  }
  vol = v;
  inCont = ic;
  outCont = oc;
}

// Which of the four slab-size classes a plan uses: bit i of c set = split rank i has its larger slab.
inline bool classUsed(const cuttHipPackedArgs& a, int c) {
  return !((c & 1) && a.split[0].slabRem == 0) && !((c & 2) && a.split[1].slabRem == 0);
}

// Threads per workgroup and elements per lane (1, 2, 4, 8, 16) for a staged block of `vol`
// elements.  numThreads = 0: does not fit.  A lane keeps three table words and the data of each of
// its elements in registers; 64 bytes of data per lane (8 x 8 bytes or 16 x 4 bytes) is the most
// that fits 128 registers, the budget of a 1024-lane workgroup.
inline int maxElemsPerThread(int elemSize) { return elemSize == 4 ? 16 : 8; }

void choosePackedThreads(int64_t vol, int elemSize, const cuttHipDeviceProps& props, int opt_e, int& numThreads,
                         int& elemsPerThread) {
  const int kMaxElemsPerThread = maxElemsPerThread(elemSize);
  numThreads = 0;
  elemsPerThread = 0;
  // As many elements per lane as the block allows: the loads a lane has in flight are what hides
  // the memory latency, and smaller workgroups leave room for more of them on a CU.
  int e = opt_e > 0 ? std::min(opt_e, kMaxElemsPerThread) : (vol >= 512 ? 8 : (vol >= 256 ? 4 : (vol > 64 ? 2 : 1)));
  while (e < kMaxElemsPerThread && roundUp64(ceilDiv(vol, e)) > props.maxThreadsPerBlock) e *= 2;
  const int64_t nt = roundUp64(ceilDiv(vol, e));
  if (nt > props.maxThreadsPerBlock) return;
  numThreads = (int)nt;
  elemsPerThread = e;
}

// Lanes of the packed kernel that fit a CU: 512 registers per SIMD lane in units of 8, 4 SIMDs of
// 64-lane wavefronts, at most 8 wavefronts per SIMD.
int64_t packedThreadsPerCU(const cuttHipDeviceProps& props, int elemSize, int elemsPerThread, int wide) {
  const int regs = cuttHipPackedRegsPerLane(elemSize, elemsPerThread, wide);
  int64_t t = props.maxThreadsPerCU;
  if (regs > 0) t = std::min<int64_t>(t, 4 * 64 * std::min(8, 512 / ((regs + 7) / 8 * 8)));
  return t;
}

// True if the input runs of a packed candidate are at most four 128-byte lines long and do not all
// start on a line: every stride that moves a run's start - the other ranks of the block, the slab
// step of a cut rank, the Mbar ranks - would have to be a whole number of lines.
bool shortUnalignedInputRuns(const Split& sp, const Problem& pb, const cuttHipPackedArgs& a) {
  int64_t inCont = 0;
  for (int c = 0; c < 4; c++)
    if (classUsed(a, c)) inCont = std::max<int64_t>(inCont, a.cls[c].inCont);
  if (inCont * pb.elemSize > 512) return false;
  const int64_t lineElems = 128 / pb.elemSize;
  bool prefix = true;
  for (int r = 0; r < pb.rank; r++) {
    const int slot = sp.splitSlot(r);
    if (slot >= 0) {
      // slabs start slabFloor entries apart (and one more where the extent does not divide)
      const int64_t step = (int64_t)a.split[slot].slabFloor * pb.strideIn[r];
      if (step % lineElems != 0 || (a.split[slot].slabRem && pb.strideIn[r] % lineElems != 0)) return true;
    }
    const bool inRun = prefix && sp.inMmk[r];
    if (!inRun && pb.dim[r] > 1 && pb.strideIn[r] % lineElems != 0) return true;
    if (!sp.inMmk[r] || slot >= 0 || pb.gapIn[r]) prefix = false;
  }
  return false;
}

// Number the work items of a packed plan by a list of digits (fastest first; which 0 / 1 = slab of the first /
// second cut rank, 2 = Mbar position; each digit advances its coordinate by its weight).  Needs no kernel
// support: a work item's offsets are linear in every digit as long as all slabs of a cut rank have one size,
// so the digits become the entries of the table that the kernel decodes an item number with (the Mbar table:
// extent = radix, strides = what one step of the digit adds to the two offsets), the cut ranks' slab counts
// become 1 and the table's positions the work items.  False (and nothing changed) if a cut rank has slabs of
// two sizes, if the digits of a coordinate are no mixed-radix number of exactly its extent, or if an Mbar digit
// straddles two ranks.
bool numberItemsByDigits(cuttHipPackedArgs& a, const cuttHipTileDigits& dg) {
  if (a.split[0].slabRem || a.split[1].slabRem || dg.n < 1) return false;
  const int64_t extent[3] = {a.split[0].numSplit, a.split[1].numSplit, a.volMbar};
  for (uint32_t w = 0; w < 3; w++) {  // per coordinate: weights 1, r1, r1*r2, ... up to the extent
    int64_t span = 1;
    for (;;) {
      int next = -1;
      for (int i = 0; i < dg.n; i++)
        if (dg.d[i].which == w && dg.d[i].radix > 1 && (int64_t)dg.d[i].weight == span) next = next < 0 ? i : -2;
      if (next == -1) break;
      if (next < 0) return false;  // two digits of one weight
      span *= dg.d[next].radix;
    }
    int64_t all = 1;
    for (int i = 0; i < dg.n; i++)
      if (dg.d[i].which == w && dg.d[i].radix > 1) all *= dg.d[i].radix;
    if (span != all || span != extent[w]) return false;
  }
  cuttHipMbar mb;
  std::memset(&mb, 0, sizeof(mb));
  int64_t items = 1;
  for (int i = 0; i < dg.n; i++) {
    const cuttHipTileDigit& d = dg.d[i];
    if (d.radix <= 1) continue;
    if (mb.n >= CUTT_MAX_RANK) return false;
    int64_t stepIn = 0, stepOut = 0;
    if (d.which < 2) {
      const cuttHipSplitRank& sr = a.split[d.which];
      stepIn = (int64_t)d.weight * sr.slabFloor * (int64_t)sr.strideIn;
      stepOut = (int64_t)d.weight * sr.slabFloor * (int64_t)sr.strideOut;
    } else {
      int64_t below = 1;
      int k = 0;
      for (; k < a.mbar.n; below *= a.mbar.d[k].extent, k++)
        if ((int64_t)d.weight >= below && (int64_t)d.weight < below * a.mbar.d[k].extent) break;
      if (k == a.mbar.n || (int64_t)d.weight % below != 0) return false;
      const int64_t u = (int64_t)d.weight / below;
      if ((int64_t)a.mbar.d[k].extent % (u * d.radix) != 0) return false;  // the digit stays inside rank k
      stepIn = u * (int64_t)a.mbar.d[k].strideIn;
      stepOut = u * (int64_t)a.mbar.d[k].strideOut;
    }
    if (stepIn > 0xffffffffll || stepOut > 0xffffffffll) return false;
    mb.d[mb.n].extent = d.radix;
    mb.d[mb.n].strideIn = (uint32_t)stepIn;
    mb.d[mb.n].strideOut = (uint32_t)stepOut;
    mb.n++;
    items *= d.radix;
  }
  if (mb.n < 1 || items > 0x7fffffffll || cuttHipFinishMbar(&mb) != 0) return false;
  a.mbar = mb;
  a.volMbar = (int)items;
  for (int i = 0; i < 2; i++) {
    a.split[i].numSplit = 1;
    a.split[i].strideIn = a.split[i].strideOut = 0;
    a.split[i].div = cuttHipMakeDivisor(1);
  }
  a.itemOrder = 0;
  return true;
}

// Address bit 11 among the work items that run together.
//
// Measured (150 random orders of the binary digits of slab and Mbar indices on each of 30 packed
// candidates of eight tensors with power-of-two extents, 1.3e8-2.7e8 elements of both widths; rates from
// 2.8 to 5.9 TB/s on one candidate): one thing stands out of the noise on every candidate, the same that
// the tiled kernel shows (addressBitOrder).  The digit that moves the read or the written address by 2 KB
// must not sit where it is constant for everything in flight: at the positions between the digits that
// the resident workgroups of an XCD differ in and the three slowest digits, which the eight XCDs split
// among them - all XCDs walk their chunks at the same pace, so such a digit has one value on the whole
// chip for thousands of work items - it costs 10-20 % (write side) or 5-15 % (read side); any other place
// is fine, no other digit shows more than the +-5 % of the timing noise.  So: the default numbering (slabs
// of the first cut rank, of the second, Mbar ranks), with the digits at bit 11 that would lie in that zone
// moved to the very top.  `residentPerXcd` = workgroups one XCD holds at a time.  False if there is nothing
// to move (or the numbering cannot be written as at most 16 digits).
bool thawAddressBit11(const cuttHipPackedArgs& a, int elemSize, int64_t residentPerXcd, cuttHipTileDigits& dg) {
  if (a.split[0].slabRem || a.split[1].slabRem) return false;
  auto log2Exact = [](int64_t v) {
    int l = 0;
    while ((int64_t{1} << l) < v) l++;
    return (int64_t{1} << l) == v ? l : -1;
  };
  const int esBits = elemSize == 8 ? 3 : 2;
  struct Part {
    uint32_t which;
    int64_t radix, weight;
    bool bit11;
  };
  std::vector<Part> seq;
  // one entry of the default numbering: a coordinate's rank of `extent` positions, `weight` apart in the
  // coordinate, whose step moves the two addresses by stepIn / stepOut elements; cut at its bit-11 digit(s)
  auto add = [&](uint32_t which, int64_t extent, int64_t weight, int64_t stepIn, int64_t stepOut) {
    if (extent <= 1) return;
    int cut[2] = {-1, -1};
    int n = 0;
    for (int64_t step : {stepIn, stepOut}) {
      const int l = step > 0 ? log2Exact(step) : -1;
      const int t = l < 0 ? -1 : 11 - esBits - l;  // the binary digit of this rank that moves byte-address bit 11
      if (t >= 0 && extent % (int64_t{1} << (t + 1)) == 0 && t != cut[0]) cut[n++] = t;
    }
    if (n == 2 && cut[0] > cut[1]) std::swap(cut[0], cut[1]);
    int64_t done = 1;  // positions of the rank covered so far
    for (int i = 0; i < n; i++) {
      const int64_t lowRadix = (int64_t{1} << cut[i]) / done;
      if (lowRadix > 1) seq.push_back({which, lowRadix, weight * done, false});
      seq.push_back({which, 2, weight << cut[i], true});
      done = int64_t{1} << (cut[i] + 1);
    }
    if (extent / done > 1) seq.push_back({which, extent / done, weight * done, false});
  };
  for (uint32_t i = 0; i < 2; i++)
    add(i, a.split[i].numSplit, 1, (int64_t)a.split[i].slabFloor * a.split[i].strideIn, (int64_t)a.split[i].slabFloor * a.split[i].strideOut);
  int64_t below = 1;
  for (int k = 0; k < a.mbar.n; k++) {
    add(2, a.mbar.d[k].extent, below, a.mbar.d[k].strideIn, a.mbar.d[k].strideOut);
    below *= a.mbar.d[k].extent;
  }
  double total = 0;
  for (const Part& p : seq) total += std::log2((double)p.radix);
  const double inFlight = std::log2((double)std::max<int64_t>(1, a.itemsPerBlock)) + std::log2((double)std::max<int64_t>(1, residentPerXcd));
  std::vector<Part> kept, moved;
  double pos = 0;
  for (const Part& p : seq) {
    // (half a digit of margin on the fast side: a digit that only part of the resident workgroups differ in)
    if (p.bit11 && pos >= inFlight - 0.5 && pos < total - 3.0) moved.push_back(p);
    else kept.push_back(p);
    pos += std::log2((double)p.radix);
  }
  if (moved.empty() || kept.size() + moved.size() > CUTT_MAX_TILE_DIGITS) return false;
  std::memset(&dg, 0, sizeof(dg));
  kept.insert(kept.end(), moved.begin(), moved.end());
  for (const Part& p : kept) {
    if (p.radix > 0x7fffffffll || p.weight > 0x7fffffffll) return false;
    cuttHipTileDigit& o = dg.d[dg.n++];
    o.which = p.which;
    o.radix = (uint32_t)p.radix;
    o.weight = (uint32_t)p.weight;
    o.div = cuttHipMakeDivisor((uint32_t)p.radix);
  }
  return true;
}

// Fill the launch geometry of a Packed / PackedSplit candidate.  False = does not fit.
bool setupPacked(Plan& plan, const cuttHipDeviceProps& props, const PlannerOptions& opt) {
  const Split& sp = plan.split;
  const Problem& pb = plan.pb;
  cuttHipPackedArgs& a = plan.packed;
  std::memset(&a, 0, sizeof(a));
  a.elemSize = pb.elemSize;
  a.volMbar = (int)sp.volMbar;
  a.padShift = opt.padShift > 0 ? opt.padShift : kPadShift;
  a.cachePolicy = opt.cachePolicy;
  // what bounds the offsets is the span: a piece of a larger tensor reaches further than its volume
  a.volume = pb.span;
  a.wideOffsets = (opt.wideOffsets || (uint64_t)pb.span * (uint64_t)pb.elemSize > (1ull << 32)) ? 1 : 0;
  for (int i = 0; i < 2; i++) {
    cuttHipSplitRank& sr = a.split[i];
    sr.numSplit = 1;
    if (sp.method == kPackedSplit && sp.splitRank[i] >= 0) {
      sr.numSplit = sp.numSplit[i];
      sr.slabFloor = sp.splitDim[i] / sp.numSplit[i];
      sr.slabRem = sp.splitDim[i] % sp.numSplit[i];
      sr.strideIn = (uint32_t)pb.strideIn[sp.splitRank[i]];
      sr.strideOut = (uint32_t)pb.strideOut[sp.splitRank[i]];
      if (sr.slabFloor < 1) return false;
    }
    sr.div = cuttHipMakeDivisor((uint32_t)sr.numSplit);
  }
  for (int c = 0; c < 4; c++) {
    if (!classUsed(a, c)) continue;
    const int slab[2] = {a.split[0].slabFloor + (c & 1), a.split[1].slabFloor + ((c >> 1) & 1)};
    int64_t vol, ic, oc;
    classGeometry(sp, pb, slab, vol, ic, oc);
    if (vol > kMaxLdsSlots) return false;
    cuttHipPackedClass& k = a.cls[c];
    k.vol = (int)vol;
    k.inCont = (int)ic;
    k.outCont = (int)oc;
    k.inDiv = cuttHipMakeDivisor((uint32_t)ic);
    k.outDiv = cuttHipMakeDivisor((uint32_t)oc);
    a.maxVol = std::max(a.maxVol, k.vol);
  }
  const int64_t slots = paddedSlots(a.maxVol, a.padShift);
  if (slots > kMaxLdsSlots) return false;
  a.ldsElems = (int)slots;
  plan.ldsBytes = cuttHipPackedLdsBytes(&a);
  if (plan.ldsBytes > props.ldsPerBlock) return false;
  choosePackedThreads(a.maxVol, pb.elemSize, props, opt.elemsPerThread, a.numThreads, a.elemsPerThread);
  if (a.numThreads == 0) return false;
  // Work items per workgroup: amortise the table load without starving the chip of workgroups.
  const int64_t items = sp.volMbar * (int64_t)a.split[0].numSplit * a.split[1].numSplit;
  if (items > 0x7fffffffll) return false;
  const int64_t residentPerCU =
      std::max<int64_t>(1, std::min<int64_t>((int64_t)(props.ldsPerCU / plan.ldsBytes),
                                             packedThreadsPerCU(props, pb.elemSize, a.elemsPerThread, a.wideOffsets) /
                                                 a.numThreads));
  // Enough workgroups for several waves of residents, but several items each where possible: the
  // table slice a workgroup loads is reused by all of its items.
  if (opt.packedRounds > 0) {
    // exactly `packedRounds` waves of resident workgroups, each with an equal share of the items
    const int64_t target = (int64_t)props.cuCount * residentPerCU * opt.packedRounds;
    a.itemsPerBlock = (int)std::max<int64_t>(1, ceilDiv(items, target));
  } else {
    const int64_t wanted = (int64_t)props.cuCount * residentPerCU * 4;
    // Measured on 200M-element tensors: with 8-byte elements and items of 10 KB and more, two items
    // per workgroup run about 2 % faster than four (the table is a smaller share of the traffic and
    // more workgroups even out the tail); with 4-byte elements four is better.
    const int64_t maxItems = opt.maxItemsPerBlock > 0 ? opt.maxItemsPerBlock
                             : (pb.elemSize == 8 && plan.ldsBytes >= 10 * 1024) ? 2 : 4;
    a.itemsPerBlock = (int)std::max<int64_t>(1, std::min<int64_t>(maxItems, items / std::max<int64_t>(wanted, 1)));
  }
  // (workgroups x lanes must fit a 32-bit count: more items per workgroup if they would not)
  const int64_t maxBlocks = (int64_t)(CUTT_HIP_MAX_GRID_LANES / (uint64_t)a.numThreads) - kNumXcd;
  if (ceilDiv(items, a.itemsPerBlock) > maxBlocks) a.itemsPerBlock = (int)ceilDiv(items, maxBlocks);
  // A workgroup that walks neighbouring slabs of two sizes reloads its table entries whenever the
  // size changes, about 1.2 us each time (measured: candidates ran 10-20 % behind their estimate
  // once that happened at more than one item in ten).  Such a plan lets every workgroup keep its
  // slabs and walk Mbar positions instead; the neighbouring slabs go to the neighbouring workgroups.
  {
    const double ns0 = a.split[0].numSplit, ns1 = a.split[1].numSplit;
    const double changes = (a.split[0].slabRem ? 2.0 / ns0 : 0.0) + (a.split[1].slabRem ? 2.0 / (ns0 * ns1) : 0.0);
    a.itemOrder = opt.itemOrder >= 0 ? opt.itemOrder : (changes > 0.1 && a.itemsPerBlock > 1 && sp.volMbar > 1 ? 1 : 0);
    // Input runs of at most four lines that start off the 128-byte grid share their first and last line
    // with the neighbouring slab's runs.  A workgroup that walks neighbouring slabs one after the other
    // asks for those lines twice, microseconds apart; when the neighbouring slabs run at the same time
    // in neighbouring workgroups the two requests meet in the L2.  Measured on the plans cuttPlan picks
    // for random tensors of 2e8 4-byte elements, every setting timed on the same candidate: on some
    // MI355X boxes such plans run 10-25 % behind their estimate under order 0 and order 2 brings them
    // back (32 plans: +10 % in the mean, -2 ... +22 %; one item per workgroup +6.5 %, -14 ... +24 %;
    // order 1 +11 % but down to -29 % on other plans, where order 2 is neutral); on other boxes order 0
    // already runs at the estimate and order 2 changes nothing (47 plans: -0.5 ... +1.9 % in the mean).
    // With 8-byte elements the gain was +2.8 % on the first kind of box and -2.5 % on the second (28 changed
    // plans): left as it is.
    // (Tensors that fit the memory-side cache keep order 0: three of about 5e7 elements ran 5-8 % slower
    // under order 2.)
    const double cacheBytes = props.infinityCacheBytes > 0 ? (double)props.infinityCacheBytes : 256.0 * 1024 * 1024;
    if (opt.itemOrder < 0 && a.itemOrder == 0 && a.itemsPerBlock > 1 && pb.elemSize == 4 &&
        (double)pb.volume * pb.elemSize > cacheBytes && shortUnalignedInputRuns(sp, pb, a))
      a.itemOrder = 2;
    if (a.itemOrder == 1) {
      a.itemsPerBlock = (int)std::min<int64_t>(a.itemsPerBlock, sp.volMbar);
      const int64_t slabs = (int64_t)a.split[0].numSplit * a.split[1].numSplit;
      if (ceilDiv(sp.volMbar, a.itemsPerBlock) * slabs > maxBlocks) a.itemOrder = 0;
    }
  }
  if (!fillMbar(pb, sp.inMmk, opt.mbarOrder, a.mbar)) return false;
  std::memset(&plan.itemDigits, 0, sizeof(plan.itemDigits));
  if (!opt.itemDigits.empty() && opt.itemOrder < 0) {
    cuttHipTileDigits dg;
    // (a text whose radices do not multiply to the extents is ignored)
    if (parseTileDigits(opt.itemDigits, a.split[0].numSplit, a.split[1].numSplit, sp.volMbar, dg) == items && numberItemsByDigits(a, dg))
      plan.itemDigits = dg;
  } else if (opt.addressBits && opt.itemOrder < 0 && a.itemOrder == 0 && opt.xcdAware) {
    const double cacheBytes = props.infinityCacheBytes > 0 ? (double)props.infinityCacheBytes : 256.0 * 1024 * 1024;
    cuttHipTileDigits dg;
    if ((double)pb.volume * pb.elemSize > 0.75 * cacheBytes &&
        thawAddressBit11(a, pb.elemSize, (int64_t)props.cuCount / kNumXcd * residentPerCU, dg) && numberItemsByDigits(a, dg))
      plan.itemDigits = dg;
  }
  const int64_t numbers = cuttHipPackedItemNumbers(&a);
  if (numbers < 1) return false;
  plan.numBlocks = ceilDiv(numbers, a.itemsPerBlock);
  if (opt.xcdAware && plan.numBlocks >= 64) {
    a.xcdChunk = (uint32_t)ceilDiv(plan.numBlocks, kNumXcd);
    plan.numBlocks = (int64_t)a.xcdChunk * kNumXcd;
  }
  plan.numThreads = a.numThreads;
  return true;
}

// Ordering of a tiled launch: fills order, super-tile shape and the per-XCD chunk; returns the
// number of workgroups.
struct TileOrdering {
  int order;
  uint32_t xcdChunk, superM, superK;
};

// Order 7: the digits of `text` ("m2,k8,b0,m0,k0": coordinate letter + radix, fastest first; radix 0 = what
// is left of the coordinate; "m2@4" gives the digit the weight 4 in its coordinate instead of the product of
// the coordinate's earlier radices).  A coordinate whose digits do not reach its extent gets one more,
// slowest, digit.  Returns the number of logical workgroups, 0 if the text is malformed.
int64_t parseTileDigits(const std::string& text, int64_t tilesM, int64_t tilesK, int64_t volMbar, cuttHipTileDigits& dg) {
  std::memset(&dg, 0, sizeof(dg));
  const int64_t extent[3] = {tilesM, tilesK, volMbar};
  int64_t span[3] = {1, 1, 1};
  auto push = [&](int which, int64_t radix, int64_t weight) {
    if (radix == 1) return true;
    if (dg.n >= CUTT_MAX_TILE_DIGITS || radix < 1 || radix > 0x7fffffffll || weight < 1 || weight > 0x7fffffffll) return false;
    dg.d[dg.n].which = (uint32_t)which;
    dg.d[dg.n].radix = (uint32_t)radix;
    dg.d[dg.n].weight = (uint32_t)weight;
    dg.d[dg.n].div = cuttHipMakeDivisor((uint32_t)radix);
    dg.n++;
    span[which] *= radix;
    return true;
  };
  auto number = [&](size_t& pos) {
    int64_t v = 0;
    while (pos < text.size() && text[pos] >= '0' && text[pos] <= '9') v = v * 10 + (text[pos++] - '0');
    return v;
  };
  size_t pos = 0;
  while (pos < text.size()) {
    const char c = text[pos++];
    const int which = c == 'm' ? 0 : (c == 'k' ? 1 : (c == 'b' ? 2 : -1));
    if (which < 0) return 0;
    int64_t radix = number(pos), weight = span[which];
    if (pos < text.size() && text[pos] == '@') {
      pos++;
      weight = number(pos);
    }
    if (pos < text.size() && text[pos] == ',') pos++;
    if (radix == 0) radix = ceilDiv(extent[which], span[which]);
    if (!push(which, radix, weight)) return 0;
  }
  for (int w : {2, 0, 1})
    if (span[w] < extent[w] && !push(w, ceilDiv(extent[w], span[w]), span[w])) return 0;
  if (dg.n == 0) {  // a single workgroup
    dg.d[0].which = 0; dg.d[0].radix = 1; dg.d[0].weight = 1; dg.d[0].div = cuttHipMakeDivisor(1); dg.n = 1;
  }
  int64_t logical = 1;
  for (int i = 0; i < dg.n; i++) {
    logical *= dg.d[i].radix;
    if (logical > 0x7fffffffll) return 0;
  }
  return logical;
}

// What the ordering rules of a tiled launch look at.
struct TiledShape {
  int64_t tilesM = 1, tilesK = 1, volMbar = 1;
  int64_t volMmLastTile = kTile;            // elements along Mm in the last tile
  int64_t rowBytesIn = 0, rowBytesOut = 0;  // bytes of one row of the Mm / Mk axis (0: not known, TiledCopy)
  int elemSize = 4;
  bool mbarBetween = false;        // an Mbar rank follows Mm in the input and Mk in the output
  bool beyondCache = false;        // more than 0.75 memory-side cache sizes per buffer
  bool neighbourRunsInMm = false;  // a fused Mm axis of which one rank follows Mk in the output
  bool oneRankMk = false;          // a single rank along Mk
};

int64_t tiledBlocks(const PlannerOptions& opt, const TiledShape& shape, TileOrdering& o, cuttHipTileDigits& dg) {
  const int64_t tilesM = shape.tilesM, tilesK = shape.tilesK, volMbar = shape.volMbar, volMmLastTile = shape.volMmLastTile;
  const int64_t rowBytesIn = shape.rowBytesIn, rowBytesOut = shape.rowBytesOut;
  const int elemSize = shape.elemSize;
  const bool mbarBetween = shape.mbarBetween, beyondCache = shape.beyondCache, neighbourRunsInMm = shape.neighbourRunsInMm,
             oneRankMk = shape.oneRankMk;
  std::memset(&dg, 0, sizeof(dg));
  if (!opt.tileDigits.empty()) {
    const int64_t logical = parseTileDigits(opt.tileDigits, tilesM, tilesK, volMbar, dg);
    if (logical > 0) {
      o.order = 7;
      o.superM = o.superK = 1;
      o.xcdChunk = 0;
      if (opt.xcdAware && logical >= 64) {
        const int64_t chunk = ceilDiv(logical, kNumXcd);
        if (chunk * kNumXcd <= 0x7fffffffll) {
          o.xcdChunk = (uint32_t)chunk;
          return chunk * kNumXcd;
        }
      }
      return logical;
    }
  }
  // Default: strips of super-tiles, each strip visited for all Mbar positions in turn (order 5;
  // with one Mbar position that is order 3).  The runs of consecutive Mbar positions are usually
  // neighbours in memory, so their shared lines meet in the L2: against finishing one Mbar position
  // after the other, (192,270,27,110)/(3,2,0,1) fp64 went from 3.5 to 4.8 TB/s, C4's Tiled plan from
  // 5.05 to 5.4 TB/s, and nothing measured got slower.
  o.order = opt.tiledOrder >= 0 ? opt.tiledOrder : (volMbar > 1 ? 5 : 3);
  // ... unless the Mm axis runs over fused ranks of which one follows Mk in the output: the runs that are
  // neighbours in the output then belong to other rows of the Mm axis, not to the next Mbar position, and
  // all strips along Mm should pass before the Mbar position moves on (order 3).  Six 8-byte tensors of the
  // reference's suites whose fused-Mm plan has one or two tiles along Mk: 1015-1257 us in order 5,
  // 772-862 us in order 3 (554 against 802, 561 against 769 us on two more); a seventh lost 9 %.
  if (opt.tiledOrder < 0 && neighbourRunsInMm) o.order = 3;
  // ... and with every row on the 128-byte grid on both sides (no line is shared, the strips have nothing to keep
  // together) such a plan walks the whole Mm axis at a stretch, order 1: 50 seeded plans of 0.3-0.8 GB per buffer in
  // two sets (extents with and without powers of two, both widths, with and without Mbar ranks) ran +3.2 % in the
  // mean against the strips, -1.8 % at worst; the tiles along Mk fastest +2 % (-6 ... +14 %), order 5 -0.5 %.
  // (All of those with a single rank along Mk; of two plans with a fused Mk axis one lost 10 %: left to the strips.)
  if (opt.superAuto && opt.tiledOrder < 0 && neighbourRunsInMm && oneRankMk && beyondCache && rowBytesIn > 0 &&
      rowBytesIn % 128 == 0 && rowBytesOut % 128 == 0)
    o.order = 1;
  // One measured exception (forced-Tiled sweep over random shapes, all orders timed): with two
  // tiles along Mm of which the second is thin (a 65..88-wide rank), the tiles along Mk should run
  // fastest (order 2: 10-25 % faster), so that the thin tiles' few output rows are written as
  // streams - as long as the two tiles that share an input row stay close (at most 64 tiles along Mk).
  // With 4-byte elements that holds up to a 104-wide rank (ten three-rank tensors with a leading rank of
  // 89..104, batches and reversals: +1 ... +21 %, all ten faster; a second set of 24 on another box: +3 % in
  // the mean, -9 ... +8 %, 19 faster; 110..126 wide: -7 ... +4 %; 8-byte elements beyond 88: +2 % in the
  // mean, left alone).
  if (opt.tiledOrder < 0 && tilesM == 2 && tilesK >= 3 && tilesK <= 64 && volMmLastTile <= (elemSize == 4 ? 40 : 24))
    o.order = 2;
  // Matrices, and batches of separate matrices, whose rows lie on the 128-byte grid on both sides: no tile shares
  // a line with another, and what a row of tiles along Mk writes - 64 output rows - is one contiguous piece of
  // memory.  With the tiles along Mk running fastest (order 2) the output is written front to back.  Measured
  // on forced Tiled plans of 180 random such matrices of 0.25-1.6 GB in three seeded sets (extents multiples of
  // 64, both widths, batches of 2-8), against the strips: +4 % in the mean with 17-700 tiles along Mk and 16 and
  // more along Mm (most between -2 and +9 %; one -15 %, one +23 %), nothing outside those limits (16 tiles and
  // fewer +0.8 %, beyond 700 +0.3 %).  Not when the input rows are a multiple of 4 KB apart or within 1 KB of
  // a multiple of 16 KB: the 64 rows a tile reads then fall into few memory channels, and a band that spans the
  // whole of Mk has nothing else in flight (-8 ... -10 % at multiples of 32 and 64 KB); and not off the line
  // grid, where the tiles that share lines along Mm must run together (40 matrices: -6 % in the mean).
  // Mbar ranks anywhere but between Mm and Mk: +4.2 % over 30 seeded plans of ranks 3-5 (-10 ... +15 %).  With a
  // rank between, a band of 64 output rows is no contiguous piece; three seeded sets of such plans read +1.9 %,
  // +5.5 % and -0.4 % (-15 % at worst) against the patches and strips below, which they keep.
  if (opt.superAuto && opt.tiledOrder < 0 && (o.order == 3 || o.order == 5) && !mbarBetween && !neighbourRunsInMm && beyondCache &&
      rowBytesIn > 0 && rowBytesIn % 128 == 0 && rowBytesOut % 128 == 0 && tilesM >= 16 && tilesK >= 17 && tilesK <= 700 &&
      rowBytesIn % 4096 != 0 && rowBytesIn % 16384 >= 1024 && rowBytesIn % 16384 <= 16384 - 1024)
    o.order = 2;
  // Super-tiles of up to superM x superK tiles, shrunk where a direction has fewer tiles.
  int64_t superM = opt.superM, superK = opt.superK;
  bool gridRule = false;
  if (opt.superAuto && o.order == 5) {
    // Strips that run through all of Mk keep the tiles that share a partly covered line close
    // together.  When all rows start and end on the 128-byte grid on both sides no line is shared
    // between tiles, and patches that are short along Mk bring the next Mbar position back sooner, which
    // pays when that position is the neighbouring row of the same matrix on both sides (an Mbar rank
    // between Mm and Mk).  Measured on forced Tiled plans of 6e7-2.6e8 8-byte elements, every shape
    // timed: patches of 8 tiles along Mk ran +2.5 % in the mean over 14 random such tensors (-1.7 %
    // ... +9 %) and +2...+6 % on five batched transposes of 1024 x 1024-like matrices with rows up
    // to 512 KB apart; two instead of eight tiles wide where Mm has 16 tiles and more gained another
    // +0.9 ... +5.7 % on five of six of the latter (one -2 %).  Outside these limits it loses: 4-byte
    // elements -3 % (worst -16 %), rows off the grid -7 %, 10 tiles along Mk cut into 5 + 5 -1...-6 %,
    // fewer than three tiles along Mm -2 %.
    // Checked again on tensors the rule was not found on (70 seeded plans with extents that are
    // multiples of 16, patches against strips in one process): with the rank between +1 % in the mean
    // over 27 (-7 ... +9 %; +4 % over ten batched transposes whose extents are multiples of 256), for
    // batches of separate matrices - the Mbar rank slowest on both sides, which used to get 8 x 8
    // patches - -1.3 % over 20 (-7 ... +3 %): those walk strips again.
    const bool onGrid = rowBytesIn % 128 == 0 && rowBytesOut % 128 == 0;
    gridRule = onGrid && elemSize == 8 && tilesK >= 16 && tilesM >= 3 && mbarBetween;
    if (gridRule) {
      superK = 8;
      // (Not two wide for input rows a multiple of 32 KB apart: ten such tensors ran 3.4 % faster 8 wide,
      // -0.6 ... +7 %.)
      if (tilesM >= 16 && rowBytesIn % 32768 != 0) superM = 2;
    }
  }
  if (opt.superAuto && (o.order == 5 || o.order == 3) && elemSize == 4 && beyondCache && rowBytesIn > 0 &&
      rowBytesIn % 32768 == 0) {
    // Input rows a multiple of 32 KB apart (8192 4-byte elements): the 64 rows a tile reads then seem to fall
    // into the same memory channels (the effect is absent at multiples of 16 KB, so the interleave would
    // repeat every 32 KB), and a strip of 8 tiles covers only 2 KB of each row.
    // Strips 16 tiles wide (4 KB per row, what 8-byte elements have anyway) measured +8 ... +15 % on forty
    // such tensors of 2e8 elements in four layouts (2-D with Mk on and off the line grid, batches, an Mbar
    // rank between; 12, 24, 32 and 64 wide and patches of 16 x 16 ... 32 x 32 all gained less), on two boxes.
    // Rows that are multiples of 4, 8 or 16 KB only: -0.3 % (-3 ... +3 %), left alone.  Tensors inside the
    // memory-side cache lose 1-5 % (8192 x 354 ... 3911); from 0.75 cache sizes per buffer on it pays.
    gridRule = true;
    superM = 16;
  }
  if (opt.superAuto && !gridRule && (o.order == 5 || o.order == 3) && tilesM > superM && tilesM <= 14 &&
      !(elemSize == 8 && rowBytesIn % 128 == 0 && rowBytesOut % 128 == 0)) {
    // A rank of 9..14 tiles is not cut into two strips (5 + 4 ... 7 + 7): one strip as wide as the rank
    // reads whole input rows.  (Up to 16 tiles at first; on 32 seeded tensors the rule was not found on, the
    // seven with 15 or 16 tiles all ran slower in one strip, -0.6 ... -9 %, the others +3 % in the mean.)  Forced Tiled plans on 13 random tensors with such a rank (both widths,
    // with and without Mbar ranks): +2.8 % in the mean, -2 % ... +8 %; the three-rank reversals of the
    // reference's bench 5 with 13 tiles along Mm and 3 along Mk, (817,1480,148)-like: 749 -> 660 us.
    // From 17 tiles on a single strip gains nothing in the mean (-7 % ... +9 %) and stays cut.  Not for
    // 8-byte rows on the line grid: (1024,64,512,6) lost 9 % with one strip of 16, (768,64,1024,4) 4 %, and
    // twenty random such tensors ran 0.9 % faster cut in two.
    superM = tilesM;
  }
  int64_t sm = std::min<int64_t>(superM, tilesM), sk = std::min<int64_t>(superK, tilesK);
  // Equal-sized super-tiles: no nearly empty last one (its padding workgroups would leave XCDs idle).
  sm = ceilDiv(tilesM, ceilDiv(tilesM, sm));
  sk = ceilDiv(tilesK, ceilDiv(tilesK, sk));
  o.superM = (uint32_t)sm;
  o.superK = (uint32_t)sk;
  int64_t logical = tilesM * tilesK * volMbar;
  if (o.order >= 3) logical = ceilDiv(tilesM, sm) * ceilDiv(tilesK, sk) * sm * sk * volMbar;
  o.xcdChunk = 0;
  if (opt.xcdAware && logical >= 64) {
    int64_t chunk = ceilDiv(logical, kNumXcd);
    if (chunk * kNumXcd <= 0x7fffffffll) {
      o.xcdChunk = (uint32_t)chunk;
      return chunk * kNumXcd;
    }
  }
  return logical;
}

// Workgroup numbering for batched transposes whose tiles sit on power-of-two addresses.
//
// Measured (random orders of the binary digits of tile and Mbar indices, 1500-2500 per tensor, on ten
// tensors of 1.6 GB per buffer, 4- and 8-byte elements): which digits change among the tiles that run
// at the same time decides 20-40 % of the rate (3.4-6.2 TB/s), and what decides is the address bit a
// digit moves, on either side, the same for every tensor:
//   - address bit 11 must differ among the tiles in flight - on the write side above all (a digit that
//     moves the written address by 2 KB, placed where it changes only every few thousand workgroups,
//     costs 10-14 %; in the three slowest digits, which the eight XCDs split among them, or among the
//     fastest seven it gains 4-6 %), the read side half as much;
//   - tile digits that move an address by 1 KB or 4 KB (bits 10, 12) and any digit that moves it by
//     128 KB (bit 17) are better left slow (3-4 % each when among the fastest four);
//   - the other digits matter little; consecutive Mbar positions and the 2 x 2 patch of tiles first.
// The rule below (bit-11 digits and one 1-KB digit slowest = split over the XCDs; 1 KB / 4 KB / 128 KB
// digits below them; 2 x 2 patch, Mbar digits, other tile digits fastest) reached 0.996 of the rate
// of the measuring planner's plan in the mean over all 35 four-rank batched transposes
// (2^a, 2^j, 2^b, 3) -> (2^b, 2^j, 2^a, 3) of 2e8 8-byte elements (lowest 0.85; the orders it replaces:
// 0.93 and 0.78), C2 5.6 -> 6.2 TB/s.  With 128 and more tiles along Mk it lost 5-14 % on five of six,
// so those keep the strips.  The same rule holds with two tiles along an axis and with tile axes over
// fused ranks (seven such tensors with an Mbar rank between Mm and Mk: +0 ... +11 % against strips and
// patches, none slower); it does not hold without such a rank, for plain 2-D transposes or with a single
// tile along an axis (-25 ... +19 %: there one side of a tile is a contiguous stream and the strips that
// keep it sequential are hard to beat), which is what the caller's conditions exclude.  Returns the
// number of logical workgroups, 0 if the tensor is not of this class.
int64_t addressBitOrder(const Problem& pb, const Split& sp, const cuttHipMbar& mb, int64_t tilesM, int64_t tilesK,
                        cuttHipTileDigits& dg) {
  auto log2Exact = [](int64_t v) {
    int l = 0;
    while ((int64_t{1} << l) < v) l++;
    return (int64_t{1} << l) == v ? l : -1;
  };
  const int es = pb.elemSize, esBits = es == 8 ? 3 : 2;
  const int bitsM = log2Exact(tilesM), bitsK = log2Exact(tilesK);
  if (bitsM < 1 || bitsK < 1 || tilesK >= 128) return 0;
  if (sp.volMm != tilesM * kTile || sp.volMk != tilesK * kTile) return 0;
  // A tile axis over fused ranks: its tiles still sit on power-of-two addresses when every rank of the set
  // has a power-of-two extent and stride; not when the output's next run starts inside the Mm set (those
  // plans walk strips per Mbar position, tiledBlocks).
  if (sp.numMm > 1 && sp.numMk < pb.rank && pb.perm[sp.numMk] > 0 && pb.perm[sp.numMk] < sp.numMm) return 0;
  // element 2^e of a fused set -> the address bit it moves on the side where the set is not contiguous
  auto otherBit = [&](int e, bool setIsMm) -> int {
    int64_t below = 1;
    const int n = setIsMm ? sp.numMm : sp.numMk;
    for (int j = 0; j < n; j++) {
      const int r = setIsMm ? j : pb.perm[j];
      const int le = log2Exact(pb.dim[r]), ls = log2Exact(setIsMm ? pb.strideOut[r] : pb.strideIn[r]);
      const int lb = log2Exact(below);
      if (le < 0 || ls < 0 || lb < 0) return -1;
      if (e < lb + le) return e - lb + ls + esBits;
      below *= pb.dim[r];
    }
    return -1;
  };
  struct Digit {
    int which, radix;
    int64_t weight;
    int rd, wr;  // address bit the digit moves on the read / write side, -1 = not a single bit
    int index;   // position among the digits of its coordinate
  };
  std::vector<Digit> all;
  for (int i = 0; i < bitsM; i++) {
    const int wr = otherBit(6 + i, true);
    if (wr < 0) return 0;
    all.push_back({0, 2, int64_t{1} << i, 6 + esBits + i, wr, i});
  }
  for (int i = 0; i < bitsK; i++) {
    const int rd = otherBit(6 + i, false);
    if (rd < 0) return 0;
    all.push_back({1, 2, int64_t{1} << i, rd, 6 + esBits + i, i});
  }
  int64_t below = 1;
  int nb = 0, binaryMbar = 0;
  for (int k = 0; k < mb.n; k++) {
    int64_t e = mb.d[k].extent, w = below;
    const int rd = log2Exact(mb.d[k].strideIn), wr = log2Exact(mb.d[k].strideOut);
    for (int t = 0; e % 2 == 0; t++, e /= 2, w *= 2) {
      all.push_back({2, 2, w, rd < 0 ? -1 : rd + esBits + t, wr < 0 ? -1 : wr + esBits + t, nb++});
      binaryMbar++;
    }
    if (e > 1) all.push_back({2, (int)e, w, -1, -1, nb++});
    below *= mb.d[k].extent;
  }
  if (binaryMbar < 2 || (int)all.size() > CUTT_MAX_TILE_DIGITS) return 0;
  auto moves = [](const Digit& d, int bit) { return d.rd == bit || d.wr == bit; };
  std::vector<Digit> top, slow, fast, odd;
  for (const Digit& d : all)
    if (d.radix == 2 && moves(d, 11)) top.push_back(d);
  auto taken = [&](const Digit& d) {
    for (const Digit& t : top)
      if (t.which == d.which && t.weight == d.weight) return true;
    return false;
  };
  if (top.size() > 3) top.resize(3);
  for (int bit : {10, 12})  // a third digit for the XCDs: a tile digit that moves 1 KB, else 4 KB
    for (const Digit& d : all)
      if (top.size() < 3 && top.size() >= 1 && d.which != 2 && d.radix == 2 && moves(d, bit) && !taken(d) &&
          (bit == 10 || top.size() == 2))
        top.push_back(d);
  for (const Digit& d : all) {
    if (taken(d)) continue;
    // (an Mbar digit that moves both addresses by 2 MB and more steps from one slice of the tensor to
    // another: among the fastest digits it cost 10-40 % on tensors whose last rank is a power of two)
    if (d.radix != 2 || (d.which == 2 && d.rd >= 21 && d.wr >= 21)) odd.push_back(d);
    else if ((d.which != 2 && (moves(d, 10) || moves(d, 12))) || moves(d, 17)) slow.push_back(d);
    else fast.push_back(d);
  }
  // fastest: the 2 x 2 patch, then the Mbar digits in their order, then the other tile digits
  std::stable_sort(fast.begin(), fast.end(), [](const Digit& a, const Digit& b) {
    auto cls = [](const Digit& d) { return d.which != 2 && d.index == 0 ? 0 : (d.which == 2 ? 1 : 2); };
    return cls(a) != cls(b) ? cls(a) < cls(b) : (cls(a) == 2 ? a.index < b.index : false);
  });
  // slowest of the slow ones: the digits that move 1 KB / 4 KB
  std::stable_sort(slow.begin(), slow.end(), [&](const Digit& a, const Digit& b) {
    const bool ka = moves(a, 10) || moves(a, 12), kb = moves(b, 10) || moves(b, 12);
    return ka != kb ? kb : a.index < b.index;
  });
  std::vector<Digit> seq = fast;
  seq.insert(seq.end(), slow.begin(), slow.end());
  // the three slowest digits are binary, so that each XCD's chunk is one value of them
  while (top.size() < 3 && !seq.empty()) {
    top.push_back(seq.back());
    seq.pop_back();
  }
  if (top.size() < 3) return 0;
  seq.insert(seq.end(), odd.begin(), odd.end());  // odd factors of the Mbar extents and far Mbar digits right below the top
  seq.insert(seq.end(), top.begin(), top.end());
  std::memset(&dg, 0, sizeof(dg));
  int64_t logical = 1;
  for (const Digit& d : seq) {
    cuttHipTileDigit& o = dg.d[dg.n++];
    o.which = (uint32_t)d.which;
    o.radix = (uint32_t)d.radix;
    o.weight = (uint32_t)d.weight;
    o.div = cuttHipMakeDivisor((uint32_t)d.radix);
    logical *= d.radix;
  }
  return logical <= 0x7fffffffll ? logical : 0;
}

bool setupTiled(Plan& plan, const cuttHipDeviceProps& props, const PlannerOptions& opt) {
  const Split& sp = plan.split;
  const Problem& pb = plan.pb;
  const int64_t tilesM = ceilDiv(sp.volMm, kTile);
  if (sp.method == kTiled) {
    cuttHipTiledArgs& a = plan.tiled;
    std::memset(&a, 0, sizeof(a));
    const int rk = pb.perm[0];
    a.elemSize = pb.elemSize;
    a.volMm = (int)sp.volMm;
    a.volMk = (int)sp.volMk;
    a.strideInK = (uint32_t)pb.strideIn[rk];
    a.strideOutM = (uint32_t)pb.strideOut[0];
    // A tile axis over several fused ranks: the rows' offsets follow the ranks' extents and strides.
    if (sp.numMm > CUTT_MAX_TILE_SET || sp.numMk > CUTT_MAX_TILE_SET || sp.volMm > 0x7fffffffll || sp.volMk > 0x7fffffffll)
      return false;
    if (sp.numMk > 1) {
      a.rowsK.n = sp.numMk;
      for (int j = 0; j < sp.numMk; j++) {
        a.rowsK.extent[j] = (uint32_t)pb.dim[pb.perm[j]];
        a.rowsK.stride[j] = (uint32_t)pb.strideIn[pb.perm[j]];
        a.rowsK.div[j] = cuttHipMakeDivisor(a.rowsK.extent[j]);
      }
    }
    if (sp.numMm > 1) {
      a.rowsM.n = sp.numMm;
      for (int r = 0; r < sp.numMm; r++) {
        a.rowsM.extent[r] = (uint32_t)pb.dim[r];
        a.rowsM.stride[r] = (uint32_t)pb.strideOut[r];
        a.rowsM.div[r] = cuttHipMakeDivisor(a.rowsM.extent[r]);
      }
    }
    a.tilesM = (int)tilesM;
    a.alignedStores = opt.tiledAligned > 0 && sp.numMm == 1 && sp.numMk == 1 ? 1 : 0;
    a.tilesK = (int)ceilDiv(sp.volMk + (a.alignedStores ? 128 / pb.elemSize - 1 : 0), kTile);
    a.volMbar = (int)sp.volMbar;
    TileOrdering o;
    // an Mbar rank that follows Mm in the input and Mk in the output: consecutive Mbar positions are
    // neighbouring rows on both sides
    bool between = false;
    for (int r = 0; r < pb.rank; r++)
      if (!sp.inMmk[r] && pb.strideIn[r] == sp.volMm && pb.strideOut[r] == sp.volMk) between = true;
    const double cacheBytes = props.infinityCacheBytes > 0 ? (double)props.infinityCacheBytes : 256.0 * 1024 * 1024;
    const bool beyondCache = (double)pb.volume * pb.elemSize > 0.75 * cacheBytes;
    if (!fillMbar(pb, sp.inMmk, opt.mbarOrder, a.mbar)) return false;
    int64_t byAddressBits = 0;
    if (opt.superAuto && opt.addressBits && opt.tiledOrder < 0 && opt.tileDigits.empty() && between && !a.alignedStores && sp.volMbar > 1 &&
        beyondCache)
      byAddressBits = addressBitOrder(pb, sp, a.mbar, a.tilesM, a.tilesK, a.digits);
    if (byAddressBits > 0) {
      o.order = 7;
      o.superM = o.superK = 1;
      o.xcdChunk = 0;
      plan.numBlocks = byAddressBits;
      if (opt.xcdAware && byAddressBits >= 64) {
        o.xcdChunk = (uint32_t)ceilDiv(byAddressBits, kNumXcd);
        plan.numBlocks = (int64_t)o.xcdChunk * kNumXcd;
      }
    } else {
      TiledShape shape;
      shape.tilesM = a.tilesM;
      shape.tilesK = a.tilesK;
      shape.volMbar = sp.volMbar;
      shape.volMmLastTile = sp.volMm - (tilesM - 1) * kTile;
      shape.rowBytesIn = sp.volMm * pb.elemSize;
      shape.rowBytesOut = sp.volMk * pb.elemSize;
      shape.elemSize = pb.elemSize;
      shape.mbarBetween = between;
      shape.beyondCache = beyondCache;
      shape.neighbourRunsInMm = sp.numMm > 1 && sp.numMk < pb.rank && pb.perm[sp.numMk] > 0 && pb.perm[sp.numMk] < sp.numMm;
      shape.oneRankMk = sp.numMk == 1;
      plan.numBlocks = tiledBlocks(opt, shape, o, a.digits);
    }
    a.order = o.order; a.xcdChunk = o.xcdChunk; a.superM = o.superM; a.superK = o.superK;
    // How the kernels decode a free numbering.  Digit by digit costs a chain of up to 16 dependent scalar loads
    // per workgroup, which a workgroup that moves a full tile hides but one that moves a quarter of it does not
    // (a (4194304,32) transpose of 4-byte elements in the digits of its default order: 4.4 TB/s digit by digit,
    // 5.8 TB/s with one digit per lane, 5.6-5.7 TB/s in the default order itself; 8-byte elements 5.1 / 5.4 /
    // 5.5).  On full tiles of 8-byte elements the lane-parallel decode is the slower one by 1-2 % (C2 6.13
    // against 6.21 TB/s, four of seven such plans; the others equal), so it is used for tiles of at most 8 KB.
    const int64_t tileBytes = std::min<int64_t>(sp.volMm, kTile) * std::min<int64_t>(sp.volMk, kTile) * pb.elemSize;
    if (a.order == 7 && (opt.digitLanes > 0 || (opt.digitLanes < 0 && tileBytes <= 8192))) cuttHipFinishTileDigits(&a.digits, &a.mbar);
    a.cachePolicy = opt.cachePolicy;
    a.grouped = opt.tiledGrouped > 0 && !a.alignedStores ? 1 : 0;  // -1: decided from the model's estimate later
    plan.ldsBytes = (size_t)(kTile + (a.alignedStores ? 128 / pb.elemSize - 1 : 0)) * (kTile + 1) * pb.elemSize;
  } else {
    cuttHipTiledCopyArgs& a = plan.tcopy;
    std::memset(&a, 0, sizeof(a));
    const int rk = pb.perm[sp.numMk - 1];
    a.elemSize = pb.elemSize;
    a.volMm = (int)sp.volMm;
    a.volMk = (int)sp.volMkBar;
    a.strideInK = (uint32_t)pb.strideIn[rk];
    a.strideOutK = (uint32_t)pb.strideOut[rk];
    a.tilesM = (int)tilesM;
    a.tilesK = (int)ceilDiv(sp.volMkBar, kTile);
    a.volMbar = (int)sp.volMbar;
    TileOrdering o;
    PlannerOptions copt = opt;
    copt.superAuto = false;  // (the measured exceptions are for the Tiled kernel only)
    TiledShape shape;
    shape.tilesM = a.tilesM;
    shape.tilesK = a.tilesK;
    shape.volMbar = sp.volMbar;
    shape.elemSize = pb.elemSize;
    plan.numBlocks = tiledBlocks(copt, shape, o, a.digits);
    a.order = o.order; a.xcdChunk = o.xcdChunk; a.superM = o.superM; a.superK = o.superK;
    a.cachePolicy = opt.cachePolicy;
    if (!fillMbar(pb, sp.inMmk, opt.mbarOrder, a.mbar)) return false;
    if (a.order == 7 && opt.digitLanes > 0) cuttHipFinishTileDigits(&a.digits, &a.mbar);
    plan.ldsBytes = 0;
  }
  plan.numThreads = 256;
  // one tile per workgroup: a tensor with tens of millions of tiny tiles has no Tiled candidate
  return plan.numBlocks <= 0x7fffffffll && (uint64_t)plan.numBlocks * 256u <= CUTT_HIP_MAX_GRID_LANES;
}

bool sameCandidate(const Split& a, const Split& b) {
  if (a.method != b.method) return false;
  switch (a.method) {
    case kTrivial: return true;
    case kTiled: return a.volMm == b.volMm && a.volMk == b.volMk && a.volMbar == b.volMbar;
    case kTiledCopy: return a.volMm == b.volMm && a.volMkBar == b.volMkBar && a.volMbar == b.volMbar;
    default:
      return a.volMmkInCont == b.volMmkInCont && a.volMmkOutCont == b.volMmkOutCont &&
             a.volStaged() == b.volStaged() && a.volMmk == b.volMmk && a.volMbar == b.volMbar;
  }
}

bool exists(const Split& s, const std::vector<Plan>& plans) {
  for (const Plan& p : plans)
    if (sameCandidate(p.split, s)) return true;
  return false;
}

bool allowed(const PlannerOptions& opt, int method) {
  return opt.forceMethod == 0 || opt.forceMethod == method;
}

void addTrivial(const Problem& red, const PlannerOptions& opt, std::vector<Plan>& plans) {
  Plan p;
  p.method = kTrivial;
  p.pb = red;
  p.fromReduced = true;
  p.split.method = kTrivial;
  p.split.update(1, 1, red);
  // one 4-KB piece per workgroup (hip_layer: cuttHipLaunchCopy)
  p.numBlocks = std::max<int64_t>(1, (red.volume * red.elemSize / 16 + 255) / 256);
  p.numThreads = 256;
  p.packed.cachePolicy = opt.cachePolicy;  // where a Trivial plan keeps its policy
  plans.push_back(std::move(p));
}

void addTiled(const Problem& red, const cuttHipDeviceProps& props, const PlannerOptions& opt,
              std::vector<Plan>& plans) {
  if (red.rank < 2) return;
  if (red.perm[0] == 0) {
    // The leading rank stays: copy rows, tile over the second output rank.
    Plan p;
    p.pb = red;
    p.fromReduced = true;
    p.method = p.split.method = kTiledCopy;
    p.split.update(1, 2, red);
    if (!allowed(opt, p.method)) return;
    if (!setupTiled(p, props, opt)) return;
    if (!exists(p.split, plans)) plans.push_back(std::move(p));
    return;
  }
  if (!allowed(opt, kTiled)) return;
  // The leading rank moves: 2-D tiles between the ranks that lead the input (Mm) and the ranks that
  // lead the output (Mk).  One rank on each side is the reference's Tiled method
  // (src/cuttplan.cpp:494-511); here either side may also run over its first two, three or four
  // ranks fused - the first numMm input ranks are one contiguous run of the input, the first numMk
  // output ranks one of the output, as long as the two sets share no rank - which the reference lists
  // as future work (README.md:197-199).  A short leading rank (36 or 166 elements) then no longer
  // leaves the 64-wide tiles half empty or cuts every row into a long and a short piece.  A side is
  // extended only while what it has so far is short (below 2048 elements, 32 tiles) and not a whole
  // number of tiles: otherwise its tiles are full anyway.
  constexpr int64_t kFuseBelow = 2048;
  const int maxSet = opt.tiledFuse == 0 ? 1 : CUTT_MAX_TILE_SET;
  int64_t volM = 1;
  for (int numMm = 1; numMm <= maxSet && numMm < red.rank; numMm++) {
    if (numMm > 1 && (volM >= kFuseBelow || volM % kTile == 0 || red.gapIn[numMm - 2])) break;
    volM *= red.dim[numMm - 1];
    int64_t volK = 1;
    for (int numMk = 1; numMk <= maxSet && numMm + numMk <= red.rank; numMk++) {
      if (numMk > 1 && (volK >= kFuseBelow || volK % kTile == 0 || red.gapOut[red.perm[numMk - 2]])) break;
      if (red.perm[numMk - 1] < numMm) break;  // the sets would share a rank (and so would every larger Mk)
      volK *= red.dim[red.perm[numMk - 1]];
      Plan p;
      p.pb = red;
      p.fromReduced = true;
      p.method = p.split.method = kTiled;
      p.split.update(numMm, numMk, red);
      if (!setupTiled(p, props, opt)) continue;
      if (!exists(p.split, plans)) plans.push_back(std::move(p));
    }
  }
}

void addPacked(const Problem& pb, bool fromReduced, const cuttHipDeviceProps& props,
               const PlannerOptions& opt, std::vector<Plan>& plans) {
  if (!allowed(opt, kPacked)) return;
  for (int numMm = 1; numMm < pb.rank; numMm++) {
    for (int numMk = 1; numMk < pb.rank; numMk++) {
      Plan p;
      p.pb = pb;
      p.fromReduced = fromReduced;
      p.method = p.split.method = kPacked;
      p.split.update(numMm, numMk, pb);
      if (p.split.volMmk > kMaxLdsSlots) break;  // larger numMk only grows the block
      if (!setupPacked(p, props, opt)) break;
      if (!exists(p.split, plans)) plans.push_back(std::move(p));
    }
  }
}

// Staged-block sizes (in elements) worth trying when Mmk has to be cut: about an eighth, a
// quarter and a half of what one workgroup's LDS holds beside its tables.
std::vector<int64_t> stagedTargets(const Problem& pb, const cuttHipDeviceProps& props) {
  // what one workgroup can stage: LDS, and the most elements its lanes can hold
  const int64_t cap = std::min<int64_t>({(int64_t)props.ldsPerBlock * 31 / 32 / pb.elemSize,
                                         (int64_t)maxElemsPerThread(pb.elemSize) * props.maxThreadsPerBlock,
                                         kMaxLdsSlots * 31 / 32});
  return {cap / 4, cap / 2, cap};
}

// Number of slabs that cuts a rank of extent `dim` into slabs of at most `slab` entries.  One
// entry of the rank spans `unit` contiguous elements; where possible the slab is rounded down so
// that unit*slab is a whole number of 128-byte lines.
int slabCount(int dim, int64_t slab, int64_t unit, int elemSize) {
  if (slab < 1) slab = 1;
  if (slab >= dim) return 1;
  const int64_t lineElems = 128 / elemSize;
  // entries per slab so that unit*entries is a multiple of a line
  int64_t step = lineElems;
  for (int64_t g = unit % lineElems; g; ) { const int64_t t = step % g; step = g; g = t; }  // gcd(unit, lineElems)
  step = lineElems / step;
  if (slab >= step) slab = slab / step * step;
  int ns = (int)ceilDiv(dim, slab);
  while (ns < dim && ceilDiv(dim, ns) > slab) ns++;
  return ns;
}

// Try one PackedSplit geometry; adds it when it fits and is new.  Returns true if it fits.
bool tryPackedSplit(const Problem& pb, bool fromReduced, const cuttHipDeviceProps& props,
                    const PlannerOptions& opt, int numMm, int numMk, int rank0, int ns0, int rank1,
                    int ns1, std::vector<Plan>& plans) {
  Plan p;
  p.pb = pb;
  p.fromReduced = fromReduced;
  p.method = p.split.method = kPackedSplit;
  int slot = 0;
  if (rank0 >= 0 && ns0 > 1) { p.split.splitRank[slot] = rank0; p.split.numSplit[slot] = ns0; slot++; }
  if (rank1 >= 0 && ns1 > 1 && rank1 != rank0) { p.split.splitRank[slot] = rank1; p.split.numSplit[slot] = ns1; slot++; }
  if (slot == 0) return false;
  p.split.update(numMm, numMk, pb);
  if (p.split.volStaged() > kMaxLdsSlots) return false;
  if (!setupPacked(p, props, opt)) return false;
  if (!exists(p.split, plans)) plans.push_back(std::move(p));
  return true;
}

void addPackedSplit(const Problem& pb, bool fromReduced, const cuttHipDeviceProps& props,
                    const PlannerOptions& opt, std::vector<Plan>& plans) {
  if (!allowed(opt, kPackedSplit)) return;
  const std::vector<int64_t> targets = stagedTargets(pb, props);
  for (int numMm = 1; numMm < pb.rank; numMm++) {
    for (int numMk = 1; numMk < pb.rank; numMk++) {
      Split base;
      base.method = kPacked;
      base.update(numMm, numMk, pb);
      // Only blocks that do not fit as one Packed block are split.
      {
        Plan probe;
        probe.pb = pb;
        probe.method = probe.split.method = kPacked;
        probe.split = base;
        if (base.volMmk <= kMaxLdsSlots && setupPacked(probe, props, opt)) continue;
      }
      bool any = false;
      // (a) Cut the largest rank of Mmk (the reference's choice, src/cuttplan.cpp:580-596).
      {
        int big = -1, maxDim = 0;
        for (int r = 0; r < numMm; r++)
          if (pb.dim[r] > maxDim) { maxDim = pb.dim[r]; big = r; }
        for (int j = 0; j < numMk; j++)
          if (pb.dim[pb.perm[j]] > maxDim) { maxDim = pb.dim[pb.perm[j]]; big = pb.perm[j]; }
        if (big >= 0 && maxDim >= 4) {
          const int64_t unsplit = base.volMmk / maxDim;
          // contiguous elements per entry of the rank, if it continues a contiguous run
          for (int64_t t : targets) {
            int64_t slab = std::max<int64_t>(2, t / std::max<int64_t>(unsplit, 1));
            slab = std::min<int64_t>(slab, maxDim / 2);
            if (slab < 2) continue;
            const int ns = slabCount(maxDim, slab, unsplit, pb.elemSize);
            if (ns >= 2 && tryPackedSplit(pb, fromReduced, props, opt, numMm, numMk, big, ns, -1, 1, plans))
              any = true;
          }
        }
      }
      // (b) Cut the last rank of the input-contiguous set and the last rank of the
      // output-contiguous set: a 2-D tile over the fused rank sets, with balanced run lengths.
      {
        const int rM = numMm - 1, rK = pb.perm[numMk - 1];
        const int dM = pb.dim[rM], dK = pb.dim[rK];
        int64_t baseIn = 1, baseOut = 1;
        for (int r = 0; r < rM; r++) baseIn *= pb.dim[r];
        for (int j = 0; j < numMk - 1; j++) baseOut *= pb.dim[pb.perm[j]];
        if (rM == rK) {
          // one rank ends both runs: covered by (a) when it is the largest; else cut it alone
          const int64_t unsplit = base.volMmk / dM;
          for (int64_t t : targets) {
            const int64_t slab = std::min<int64_t>(std::max<int64_t>(1, t / std::max<int64_t>(unsplit, 1)), dM);
            const int ns = slabCount(dM, slab, baseIn, pb.elemSize);
            if (ns >= 2 && tryPackedSplit(pb, fromReduced, props, opt, numMm, numMk, rM, ns, -1, 1, plans))
              any = true;
          }
        } else {
          const int64_t other = base.volMmk / ((int64_t)dM * dK);
          for (int64_t t : targets) {
            const double avail = (double)t / (double)other;  // budget for slabM * slabK
            if (avail < 1.0) continue;
            // Slab of the input-side rank: (0) balance the run lengths baseIn*slabM and
            // baseOut*slabK; (1), (2) keep the read runs at one or two 128-byte lines and give
            // the rest of the budget to the write runs - partly written lines cost more than
            // partly read ones, which the neighbouring workgroup finds in the L2.
            const double lineElems = 128.0 / pb.elemSize;
            const double choices[3] = {std::sqrt(avail * (double)baseOut / (double)baseIn),
                                       lineElems / (double)baseIn, 2.0 * lineElems / (double)baseIn};
            for (double sM : choices) {
              sM = std::min<double>(std::max(1.0, std::ceil(sM)), dM);
              const double sK = std::min<double>(std::max(1.0, avail / sM), dK);
              sM = std::min<double>(std::max(1.0, avail / sK), dM);
              const int nsM = slabCount(dM, (int64_t)sM, baseIn, pb.elemSize);
              const int nsK = slabCount(dK, (int64_t)sK, baseOut, pb.elemSize);
              if (nsM == 1 && nsK == 1) continue;
              if (tryPackedSplit(pb, fromReduced, props, opt, numMm, numMk, rM, nsM, rK, nsK, plans)) any = true;
            }
          }
        }
      }
      // Neither cut fits: a larger numMk only grows the block.
      if (!any) break;
    }
  }
}

}  // namespace

// Text form of a digit list (what parseTileDigits reads).
std::string formatTileDigits(const cuttHipTileDigits& dg) {
  std::string t;
  for (int i = 0; i < dg.n; i++) {
    if (i) t += ',';
    t += "mkb"[dg.d[i].which];
    t += std::to_string(dg.d[i].radix) + "@" + std::to_string(dg.d[i].weight);
  }
  return t;
}

bool rebuildPlan(const Plan& src, const cuttHipDeviceProps& props, const PlannerOptions& opt, Plan& out) {
  out = Plan();
  out.method = src.method;
  out.split = src.split;
  out.pb = src.pb;
  out.fromReduced = src.fromReduced;
  switch (src.method) {
    case kTiled:
    case kTiledCopy:
      return setupTiled(out, props, opt);
    case kPacked:
    case kPackedSplit:
      return setupPacked(out, props, opt);
    default:
      return false;
  }
}

bool createPlans(const Problem& orig, const Problem& red, const cuttHipDeviceProps& props,
                 const PlannerOptions& opt, std::vector<Plan>& plans) {
  bool identity = true;
  for (int i = 0; i < red.rank; i++) identity = identity && red.perm[i] == i;
  if (identity && red.dense) {
    // Everything fuses into one rank (or would, if the fused extent still fitted an int): a plain
    // copy is the only candidate.
    addTrivial(red, opt, plans);
    return true;
  }
  // (A piece of a larger tensor whose ranks keep their order is a copy of rows with gaps between
  // them: the TiledCopy and Packed candidates below handle it.  A single rank with gaps cannot occur:
  // a strided problem has unit strides in its leading ranks.)
  if (red.rank < 2) return false;
  addTiled(red, props, opt, plans);
  addPacked(orig, false, props, opt, plans);
  if (red.rank != orig.rank) addPacked(red, true, props, opt, plans);
  addPackedSplit(orig, false, props, opt, plans);
  if (red.rank != orig.rank) addPackedSplit(red, true, props, opt, plans);
  return true;
}

// ---------------------------------------------------------------------------
// The mixed-radix enumerations that define the index tables of slab class c: the input offsets of
// the contiguous input runs, the output offsets of the contiguous output runs, and for every
// element in output-compact order its position in input-compact order (the LDS gather, before
// padding).  False if the class geometry is inconsistent.
static bool classRadixLists(const Plan& plan, int c, std::vector<RadixDim>& rowsIn, std::vector<RadixDim>& rowsOut,
                            std::vector<RadixDim>& gather) {
  const Split& sp = plan.split;
  const Problem& pb = plan.pb;
  const cuttHipPackedArgs& packed = plan.packed;
  const int slab[2] = {packed.split[0].slabFloor + (c & 1), packed.split[1].slabFloor + ((c >> 1) & 1)};
  rowsIn.clear(); rowsOut.clear(); gather.clear();
  // Ranks of Mmk in input order with their in-compact strides.  The leading ranks up to and
  // including the first split rank form the contiguous row; the others enumerate the rows.
  std::vector<int64_t> compactIn(pb.rank, 0);
  int64_t cstride = 1;
  bool inPrefix = true;
  for (int r = 0; r < pb.rank; r++) {
    if (!sp.inMmk[r]) {
      inPrefix = false;
      continue;
    }
    const int e = blockExtent(sp, pb, r, slab);
    compactIn[r] = cstride;
    cstride *= e;
    if (!inPrefix) rowsIn.push_back({e, pb.strideIn[r]});
    if (sp.splitSlot(r) >= 0 || pb.gapIn[r]) inPrefix = false;  // ranks after a split rank or a gap start new rows
  }
  if (cstride != packed.cls[c].vol) return false;
  // Ranks of Mmk in output order.
  bool outPrefix = true;
  for (int j = 0; j < pb.rank; j++) {
    const int r = pb.perm[j];
    if (!sp.inMmk[r]) {
      outPrefix = false;
      continue;
    }
    const int e = blockExtent(sp, pb, r, slab);
    gather.push_back({e, compactIn[r]});
    if (!outPrefix) rowsOut.push_back({e, pb.strideOut[r]});
    if (sp.splitSlot(r) >= 0 || pb.gapOut[r]) outPrefix = false;
  }
  return true;
}

bool Plan::buildTables() {
  if (tablesBuilt) return true;
  if (method != kPacked && method != kPackedSplit) {
    tablesBuilt = true;
    return true;
  }
  for (int c = 0; c < 4; c++) {
    if (!classUsed(packed, c)) continue;
    PackedTables& t = tab[c];
    t.vol = packed.cls[c].vol;
    t.inCont = packed.cls[c].inCont;
    t.outCont = packed.cls[c].outCont;
    std::vector<RadixDim> rowsIn, rowsOut, gather;
    if (!classRadixLists(*this, c, rowsIn, rowsOut, gather)) return false;
    enumerateOffsets(rowsIn, t.vol / t.inCont, t.rowIn);
    enumerateOffsets(rowsOut, t.vol / t.outCont, t.rowOut);
    std::vector<uint32_t> pos;
    enumerateOffsets(gather, t.vol, pos);
    t.shIdx.resize(pos.size());
    for (size_t q = 0; q < pos.size(); q++) t.shIdx[q] = (uint16_t)(pos[q] + (pos[q] >> packed.padShift));
  }
  tablesBuilt = true;
  return true;
}

// Layout of a plan's tables in one piece of device memory: [rowIn | rowOut | shIdx] per class,
// each piece 16-byte aligned.  Returns the total size.
static size_t tableLayout(const cuttHipPackedArgs& packed, size_t off[4][3]) {
  auto align16 = [](size_t v) { return (v + 15) & ~(size_t)15; };
  size_t total = 0;
  for (int c = 0; c < 4; c++) {
    off[c][0] = off[c][1] = off[c][2] = 0;
    if (!classUsed(packed, c)) continue;
    const cuttHipPackedClass& k = packed.cls[c];
    off[c][0] = total; total += align16((size_t)(k.vol / k.inCont) * sizeof(uint32_t));
    off[c][1] = total; total += align16((size_t)(k.vol / k.outCont) * sizeof(uint32_t));
    off[c][2] = total; total += align16((size_t)k.vol * sizeof(uint16_t));
  }
  return total;
}

size_t Plan::tableBytes() const {
  if (method != kPacked && method != kPackedSplit) return 0;
  size_t off[4][3];
  return tableLayout(packed, off);
}

int Plan::activateInPlace(void* tables, size_t capacity) {
  if (method != kPacked && method != kPackedSplit) return activate();
  if (dTables || !tables) return -1;
  size_t off[4][3];
  if (tableLayout(packed, off) > capacity) return -1;
  if (int e = cuttHipPreparePacked(); e != 0) return e;
  unsigned char* base = (unsigned char*)tables;
  for (int c = 0; c < 4; c++) {
    if (!classUsed(packed, c)) continue;
    std::vector<RadixDim> lists[3];
    if (!classRadixLists(*this, c, lists[0], lists[1], lists[2])) return -1;
    cuttHipTableBuildArgs b;
    std::memset(&b, 0, sizeof(b));
    const cuttHipPackedClass& k = packed.cls[c];
    b.count[0] = (uint32_t)(k.vol / k.inCont);
    b.count[1] = (uint32_t)(k.vol / k.outCont);
    b.count[2] = (uint32_t)k.vol;
    b.padShift = packed.padShift;
    for (int l = 0; l < 3; l++) {
      if ((int)lists[l].size() > CUTT_MAX_RANK) return -1;
      b.list[l].n = (int)lists[l].size();
      for (int i = 0; i < b.list[l].n; i++) {
        b.list[l].extent[i] = (uint32_t)lists[l][i].extent;
        b.list[l].stride[i] = (uint32_t)lists[l][i].stride;
      }
    }
    b.rowIn = (uint32_t*)(base + off[c][0]);
    b.rowOut = (uint32_t*)(base + off[c][1]);
    b.shIdx = (uint16_t*)(base + off[c][2]);
    if (int e = cuttHipLaunchTableBuild(&b, stream); e != 0) return e;
    packed.cls[c].rowIn = b.rowIn;
    packed.cls[c].rowOut = b.rowOut;
    packed.cls[c].shIdx = b.shIdx;
  }
  if (int v = cuttHipValidatePacked(&packed); v != 0) return v;
  launchable = true;
  return 0;
}

int Plan::activate() {
  if (method == kTiled) return launchable ? 0 : ((launchable = cuttHipValidateTiled(&tiled) == 0) ? 0 : -1);
  if (method == kTiledCopy) return launchable ? 0 : ((launchable = cuttHipValidateTiledCopy(&tcopy) == 0) ? 0 : -1);
  if (method != kPacked && method != kPackedSplit) {
    launchable = method == kTrivial;
    return launchable ? 0 : -1;
  }
  if (dTables) return 0;
  if (!buildTables()) return -1;
  if (int e = cuttHipPreparePacked(); e != 0) return e;
  size_t off[4][3];
  const size_t total = tableLayout(packed, off);
  std::vector<unsigned char> host(total, 0);
  for (int c = 0; c < 4; c++) {
    if (!classUsed(packed, c)) continue;
    std::memcpy(&host[off[c][0]], tab[c].rowIn.data(), tab[c].rowIn.size() * sizeof(uint32_t));
    std::memcpy(&host[off[c][1]], tab[c].rowOut.data(), tab[c].rowOut.size() * sizeof(uint32_t));
    std::memcpy(&host[off[c][2]], tab[c].shIdx.data(), tab[c].shIdx.size() * sizeof(uint16_t));
  }
  void* d = nullptr;
  int e = cuttHipMalloc(&d, total);
  if (e != 0) return e;
  e = cuttHipMemcpyHtoD(d, host.data(), total);
  if (e != 0) {
    cuttHipFree(d);
    return e;
  }
  dTables = d;
  for (int c = 0; c < 4; c++) {
    if (!classUsed(packed, c)) continue;
    unsigned char* base = (unsigned char*)d;
    packed.cls[c].rowIn = (const uint32_t*)(base + off[c][0]);
    packed.cls[c].rowOut = (const uint32_t*)(base + off[c][1]);
    packed.cls[c].shIdx = (const uint16_t*)(base + off[c][2]);
  }
  if (int v = cuttHipValidatePacked(&packed); v != 0) {
    release();
    return v;
  }
  launchable = true;
  return 0;
}

int Plan::launch(const void* in, void* out) {
  if (!launchable) return -1;  // activate() checks the arguments once; launches do not repeat that
  switch (method) {
    case kTrivial:
      return cuttHipLaunchCopy(in, out, (size_t)pb.volume * pb.elemSize, packed.cachePolicy, stream);
    case kTiled:
      return cuttHipLaunchTiled(&tiled, in, out, stream);
    case kTiledCopy:
      return cuttHipLaunchTiledCopy(&tcopy, in, out, stream);
    case kPacked:
    case kPackedSplit:
      return cuttHipLaunchPacked(&packed, in, out, stream);
    default:
      return -1;
  }
}

std::string Plan::describe() const {
  std::ostringstream s;
  s << methodName(method) << (fromReduced ? " (fused ranks)" : "") << " numMm " << split.numMm
    << " numMk " << split.numMk << " volMmk " << split.volMmk << " volMbar " << split.volMbar
    << " inCont " << split.volMmkInCont << " outCont " << split.volMmkOutCont;
  if (method == kPackedSplit)
    s << " splitRank " << split.splitRank[0] << "/" << split.splitRank[1] << " numSplit " << split.numSplit[0]
      << "/" << split.numSplit[1];
  s << " blocks " << numBlocks << " threads " << numThreads << " lds " << ldsBytes;
  if (method == kPacked || method == kPackedSplit) s << " items/block " << packed.itemsPerBlock;
  s << " predicted_us " << model.usPredicted;
  return s.str();
}

}  // namespace cutt
