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
#include <cstdio>
#include <cstring>
#include <sstream>

namespace cutt {

namespace {
constexpr int kTile = 64;
constexpr int kPadShift = 5;            // one LDS pad slot per 32 elements
constexpr int64_t kMaxLdsSlots = 65536; // the gather index is 16 bits wide

inline int64_t ceilDiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int roundUp64(int64_t v) { return (int)(ceilDiv(v, 64) * 64); }
inline int64_t paddedSlots(int64_t vol) { return vol ? (vol - 1) + ((vol - 1) >> kPadShift) + 1 : 0; }
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

uint32_t divMagic(uint32_t d) {
  if (d < 2) return 0;
  return (uint32_t)(((1ull << 32) + d - 1) / d);
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
  std::strncpy(p.arch, "gfx950", sizeof(p.arch) - 1);
  return p;
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
}

void reduceRanks(int rank, const int* dim, const int* perm, std::vector<int>& redDim,
                 std::vector<int>& redPerm) {
  // Groups of output ranks whose input ranks are consecutive and increasing.
  std::vector<int> first, vol;
  for (int j = 0; j < rank; j++) {
    if (j > 0 && perm[j] == perm[j - 1] + 1) {
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
  if (splitRank >= 0) {
    splitDim = pb.dim[splitRank];
    volMmkUnsplit = volMmk / splitDim;
  } else {
    splitDim = 0;
    volMmkUnsplit = volMmk;
  }
  volMmkInCont = 1;
  for (int r = 0; r < rank && inMmk[r]; r++) {
    if (r == splitRank) {
      volMmkInCont *= slabMax();
      break;
    }
    volMmkInCont *= pb.dim[r];
  }
  volMmkOutCont = 1;
  for (int j = 0; j < rank && inMmk[pb.perm[j]]; j++) {
    const int r = pb.perm[j];
    if (r == splitRank) {
      volMmkOutCont *= slabMax();
      break;
    }
    volMmkOutCont *= pb.dim[r];
  }
}

int64_t Split::volStaged() const {
  switch (method) {
    case kPacked: return volMmk;
    case kPackedSplit: return (int64_t)slabMax() * volMmkUnsplit;
    case kTiled: return kTile * kTile;
    default: return 0;
  }
}

// ---------------------------------------------------------------------------
Plan::Plan() {
  std::memset(&tiled, 0, sizeof(tiled));
  std::memset(&tcopy, 0, sizeof(tcopy));
  std::memset(&packed, 0, sizeof(packed));
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
  ldsBytes = o.ldsBytes;
  numBlocks = o.numBlocks;
  numThreads = o.numThreads;
  tab[0] = std::move(o.tab[0]);
  tab[1] = std::move(o.tab[1]);
  tablesBuilt = o.tablesBuilt;
  dTables = o.dTables;
  o.dTables = nullptr;
  model = o.model;
  return *this;
}

void Plan::release() {
  if (dTables) {
    cuttHipFree(dTables);
    dTables = nullptr;
    for (int c = 0; c < 2; c++) {
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

void fillMbar(const Problem& pb, const std::vector<char>& inMmk, cuttHipMbar& mb) {
  std::memset(&mb, 0, sizeof(mb));
  int n = 0;
  for (int r = 0; r < pb.rank; r++) {
    if (inMmk[r]) continue;
    mb.d[n].extent = (uint32_t)pb.dim[r];
    mb.d[n].strideIn = (uint32_t)pb.strideIn[r];
    mb.d[n].strideOut = (uint32_t)pb.strideOut[r];
    n++;
  }
  mb.n = n;
}

// Extent of rank r inside one staged block of slab size `slab`.
inline int blockExtent(const Split& sp, const Problem& pb, int r, int slab) {
  return r == sp.splitRank ? slab : pb.dim[r];
}

// Geometry of one slab class: volume and contiguous run lengths.
void classGeometry(const Split& sp, const Problem& pb, int slab, int& vol, int& inCont, int& outCont) {
  int64_t v = 1, ic = 1, oc = 1;
  for (int r = 0; r < pb.rank; r++)
    if (sp.inMmk[r]) v *= blockExtent(sp, pb, r, slab);
  for (int r = 0; r < pb.rank && sp.inMmk[r]; r++) {
    ic *= blockExtent(sp, pb, r, slab);
    if (r == sp.splitRank) break;
  }
  for (int j = 0; j < pb.rank && sp.inMmk[pb.perm[j]]; j++) {
    const int r = pb.perm[j];
    oc *= blockExtent(sp, pb, r, slab);
    if (r == sp.splitRank) break;
  }
  vol = (int)v;
  inCont = (int)ic;
  outCont = (int)oc;
}

// Threads per workgroup for a staged block of `vol` elements that needs `lds` bytes.
int choosePackedThreads(int64_t vol, size_t lds, const cuttHipDeviceProps& props) {
  const int64_t byLds = std::max<int64_t>(1, (int64_t)(props.ldsPerCU / std::max<size_t>(lds, 1)));
  // Fill the CU's thread slots with the workgroups that fit by LDS ...
  int64_t nt = (props.maxThreadsPerCU / std::min<int64_t>(byLds, 8)) / 64 * 64;
  // ... but keep at least ~4 elements per lane, and stay inside the hardware limit.
  nt = std::min<int64_t>(nt, roundUp64(ceilDiv(vol, 4)));
  nt = std::min<int64_t>(nt, props.maxThreadsPerBlock);
  nt = std::max<int64_t>(nt, 64);
  return (int)nt;
}

// Fill the launch geometry of a Packed / PackedSplit candidate.  False = does not fit.
bool setupPacked(Plan& plan, const cuttHipDeviceProps& props) {
  const Split& sp = plan.split;
  const Problem& pb = plan.pb;
  cuttHipPackedArgs& a = plan.packed;
  std::memset(&a, 0, sizeof(a));
  a.elemSize = pb.elemSize;
  a.volMbar = (int)sp.volMbar;
  a.padShift = kPadShift;
  if (sp.method == kPackedSplit) {
    a.numSplit = sp.numSplit;
    a.slabFloor = sp.splitDim / sp.numSplit;
    a.slabRem = sp.splitDim % sp.numSplit;
    a.splitStrideIn = (uint32_t)pb.strideIn[sp.splitRank];
    a.splitStrideOut = (uint32_t)pb.strideOut[sp.splitRank];
    if (a.slabFloor < 1) return false;
  } else {
    a.numSplit = 1;
    a.slabFloor = 0;
    a.slabRem = 0;
  }
  const int ncls = a.slabRem > 0 ? 2 : 1;
  for (int c = 0; c < ncls; c++) {
    int vol, ic, oc;
    classGeometry(sp, pb, a.slabFloor + c, vol, ic, oc);
    cuttHipPackedClass& k = a.cls[c];
    k.vol = vol;
    k.inCont = ic;
    k.outCont = oc;
    k.inMagic = divMagic((uint32_t)ic);
    k.outMagic = divMagic((uint32_t)oc);
    k.nRowsIn = vol / ic;
    k.nRowsOut = vol / oc;
    a.maxVol = std::max(a.maxVol, vol);
    a.maxRowsIn = std::max(a.maxRowsIn, k.nRowsIn);
    a.maxRowsOut = std::max(a.maxRowsOut, k.nRowsOut);
  }
  const int64_t slots = paddedSlots(a.maxVol);
  if (slots > kMaxLdsSlots) return false;
  a.ldsElems = (int)slots;
  plan.ldsBytes = cuttHipPackedLdsBytes(&a);
  if (plan.ldsBytes > props.ldsPerBlock) return false;
  a.numThreads = choosePackedThreads(a.maxVol, plan.ldsBytes, props);
  // Work items per workgroup: amortise the table load without starving the chip of workgroups.
  const int64_t items = sp.volMbar * (int64_t)a.numSplit;
  if (items > 0x7fffffffll) return false;
  const int64_t residentPerCU =
      std::max<int64_t>(1, std::min<int64_t>((int64_t)(props.ldsPerCU / plan.ldsBytes),
                                             props.maxThreadsPerCU / a.numThreads));
  const int64_t wanted = (int64_t)props.cuCount * residentPerCU * 8;
  a.itemsPerBlock = (int)std::max<int64_t>(1, std::min<int64_t>(8, items / std::max<int64_t>(wanted, 1)));
  plan.numBlocks = ceilDiv(items, a.itemsPerBlock);
  plan.numThreads = a.numThreads;
  fillMbar(pb, sp.inMmk, a.mbar);
  return true;
}

bool setupTiled(Plan& plan, const cuttHipDeviceProps& props, const PlannerOptions& opt) {
  (void)props;
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
    a.tilesM = (int)tilesM;
    a.tilesK = (int)ceilDiv(sp.volMk, kTile);
    a.volMbar = (int)sp.volMbar;
    a.order = opt.tiledOrder >= 0 ? opt.tiledOrder : 0;
    fillMbar(pb, sp.inMmk, a.mbar);
    plan.numBlocks = (int64_t)a.tilesM * a.tilesK * sp.volMbar;
    plan.ldsBytes = (size_t)kTile * (kTile + 1) * pb.elemSize;
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
    a.order = opt.tiledOrder >= 0 ? opt.tiledOrder : 1;
    fillMbar(pb, sp.inMmk, a.mbar);
    plan.numBlocks = (int64_t)a.tilesM * a.tilesK * sp.volMbar;
    plan.ldsBytes = 0;
  }
  plan.numThreads = 256;
  return plan.numBlocks <= 0x7fffffffll;
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

void addTrivial(const Problem& red, std::vector<Plan>& plans) {
  Plan p;
  p.method = kTrivial;
  p.pb = red;
  p.fromReduced = true;
  p.split.method = kTrivial;
  p.split.update(1, 1, red);
  p.numBlocks = 1;
  p.numThreads = 1;
  plans.push_back(std::move(p));
}

void addTiled(const Problem& red, const cuttHipDeviceProps& props, const PlannerOptions& opt,
              std::vector<Plan>& plans) {
  if (red.rank < 2) return;
  Plan p;
  p.pb = red;
  p.fromReduced = true;
  if (red.perm[0] != 0) {
    // The leading rank moves: 2-D tiles between input rank 0 and the rank that leads the output.
    p.method = p.split.method = kTiled;
    p.split.update(1, 1, red);
  } else {
    // The leading rank stays: copy rows, tile over the second output rank.
    p.method = p.split.method = kTiledCopy;
    p.split.update(1, 2, red);
  }
  if (!allowed(opt, p.method)) return;
  if (!setupTiled(p, props, opt)) return;
  if (!exists(p.split, plans)) plans.push_back(std::move(p));
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
      if (!setupPacked(p, props)) break;
      if (!exists(p.split, plans)) plans.push_back(std::move(p));
    }
  }
}

// Slab counts worth trying for a block that is too large for one workgroup.
std::vector<int> splitCounts(const Split& sp, const Problem& pb, const cuttHipDeviceProps& props) {
  std::vector<int> out;
  const int64_t unsplitBytes = sp.volMmkUnsplit * pb.elemSize;
  const int splitDim = sp.splitDim;
  // Target staged sizes (data bytes): a quarter, a half and the whole of what one workgroup may hold
  // beside its tables.
  const int64_t cap = (int64_t)props.ldsPerBlock * pb.elemSize / (pb.elemSize + 3);
  const int64_t targets[3] = {cap / 8, cap / 4, cap / 2};
  for (int64_t t : targets) {
    int64_t slab = t / std::max<int64_t>(unsplitBytes, 1);
    if (slab < 2) slab = 2;
    if (slab > splitDim / 2) slab = splitDim / 2;
    if (slab < 2) continue;
    // Prefer slab sizes that cover whole 128-byte lines when the split rank is contiguous on
    // either side, and slab counts that divide the rank evenly.
    const int lineElems = 128 / pb.elemSize;
    int64_t best = slab;
    if (slab >= lineElems) best = slab / lineElems * lineElems;
    int ns = (int)ceilDiv(splitDim, best);
    // the slab the kernel uses is ceil(splitDim/ns); nudge ns so that it stays <= slab
    while (ns < splitDim && ceilDiv(splitDim, ns) > slab) ns++;
    if (ns >= 2 && std::find(out.begin(), out.end(), ns) == out.end()) out.push_back(ns);
  }
  return out;
}

void addPackedSplit(const Problem& pb, bool fromReduced, const cuttHipDeviceProps& props,
                    const PlannerOptions& opt, std::vector<Plan>& plans) {
  if (!allowed(opt, kPackedSplit)) return;
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
        if (base.volMmk <= kMaxLdsSlots && setupPacked(probe, props)) continue;
      }
      // Split the largest rank of Mmk (first one wins ties, input ranks before output ranks).
      int splitRank = -1, maxDim = 0;
      for (int r = 0; r < numMm; r++)
        if (pb.dim[r] > maxDim) { maxDim = pb.dim[r]; splitRank = r; }
      for (int j = 0; j < numMk; j++)
        if (pb.dim[pb.perm[j]] > maxDim) { maxDim = pb.dim[pb.perm[j]]; splitRank = pb.perm[j]; }
      if (splitRank < 0 || maxDim < 4) break;
      base.method = kPackedSplit;
      base.splitRank = splitRank;
      base.numSplit = 1;
      base.update(numMm, numMk, pb);
      // Even slabs of two entries must fit, otherwise larger numMk cannot fit either.
      if (paddedSlots(2 * base.volMmkUnsplit) > kMaxLdsSlots) break;
      bool any = false;
      for (int ns : splitCounts(base, pb, props)) {
        Plan p;
        p.pb = pb;
        p.fromReduced = fromReduced;
        p.method = kPackedSplit;
        p.split = base;
        p.split.numSplit = ns;
        p.split.update(numMm, numMk, pb);
        if (!setupPacked(p, props)) continue;
        any = true;
        if (!exists(p.split, plans)) plans.push_back(std::move(p));
      }
      if (!any) break;
    }
  }
}

}  // namespace

bool createPlans(const Problem& orig, const Problem& red, const cuttHipDeviceProps& props,
                 const PlannerOptions& opt, std::vector<Plan>& plans) {
  if (red.rank == 1) {
    // Everything fused into one rank: a plain copy is the only candidate.
    addTrivial(red, plans);
    return true;
  }
  addTiled(red, props, opt, plans);
  addPacked(orig, false, props, opt, plans);
  if (red.rank != orig.rank) addPacked(red, true, props, opt, plans);
  addPackedSplit(orig, false, props, opt, plans);
  if (red.rank != orig.rank) addPackedSplit(red, true, props, opt, plans);
  return true;
}

// ---------------------------------------------------------------------------
bool Plan::buildTables() {
  if (tablesBuilt) return true;
  if (method != kPacked && method != kPackedSplit) {
    tablesBuilt = true;
    return true;
  }
  const Split& sp = split;
  const int ncls = packed.slabRem > 0 ? 2 : 1;
  for (int c = 0; c < ncls; c++) {
    const int slab = packed.slabFloor + c;
    PackedTables& t = tab[c];
    t.vol = packed.cls[c].vol;
    t.inCont = packed.cls[c].inCont;
    t.outCont = packed.cls[c].outCont;
    // Ranks of Mmk in input order with their in-compact strides.
    std::vector<int64_t> compactIn(pb.rank, 0);
    int64_t cstride = 1;
    std::vector<RadixDim> rowsIn;
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
      if (r == sp.splitRank) inPrefix = false;  // ranks after the split rank start new rows
    }
    if (cstride != t.vol) return false;
    enumerateOffsets(rowsIn, t.vol / t.inCont, t.rowIn);
    // Ranks of Mmk in output order.
    std::vector<RadixDim> rowsOut, gather;
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
      if (r == sp.splitRank) outPrefix = false;
    }
    enumerateOffsets(rowsOut, t.vol / t.outCont, t.rowOut);
    std::vector<uint32_t> pos;
    enumerateOffsets(gather, t.vol, pos);
    t.shIdx.resize(pos.size());
    for (size_t q = 0; q < pos.size(); q++) t.shIdx[q] = (uint16_t)(pos[q] + (pos[q] >> packed.padShift));
  }
  tablesBuilt = true;
  return true;
}

int Plan::activate() {
  if (method != kPacked && method != kPackedSplit) return 0;
  if (dTables) return 0;
  if (!buildTables()) return -1;
  const int ncls = packed.slabRem > 0 ? 2 : 1;
  // One allocation: [rowIn | rowOut | shIdx] per class, each piece 16-byte aligned.
  auto align16 = [](size_t v) { return (v + 15) & ~(size_t)15; };
  size_t total = 0;
  size_t off[2][3];
  for (int c = 0; c < ncls; c++) {
    off[c][0] = total; total += align16(tab[c].rowIn.size() * sizeof(uint32_t));
    off[c][1] = total; total += align16(tab[c].rowOut.size() * sizeof(uint32_t));
    off[c][2] = total; total += align16(tab[c].shIdx.size() * sizeof(uint16_t));
  }
  std::vector<unsigned char> host(total, 0);
  for (int c = 0; c < ncls; c++) {
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
  for (int c = 0; c < ncls; c++) {
    unsigned char* base = (unsigned char*)d;
    packed.cls[c].rowIn = (const uint32_t*)(base + off[c][0]);
    packed.cls[c].rowOut = (const uint32_t*)(base + off[c][1]);
    packed.cls[c].shIdx = (const uint16_t*)(base + off[c][2]);
  }
  return 0;
}

int Plan::launch(const void* in, void* out) {
  switch (method) {
    case kTrivial:
      return cuttHipMemcpyDtoDAsync(out, in, (size_t)pb.volume * pb.elemSize, stream);
    case kTiled:
      return cuttHipLaunchTiled(&tiled, in, out, stream);
    case kTiledCopy:
      return cuttHipLaunchTiledCopy(&tcopy, in, out, stream);
    case kPacked:
    case kPackedSplit:
      if (!dTables) return -1;
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
    s << " splitRank " << split.splitRank << " numSplit " << split.numSplit;
  s << " blocks " << numBlocks << " threads " << numThreads << " lds " << ldsBytes;
  if (method == kPacked || method == kPackedSplit) s << " items/block " << packed.itemsPerBlock;
  s << " predicted_us " << model.usPredicted;
  return s.str();
}

}  // namespace cutt
