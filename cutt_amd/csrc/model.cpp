/*
 * model.cpp - memory-transaction cost model.  See model.h.
 *
 * The counting functions keep the reference's definitions (reference
 * src/cuttGpuModel.cpp:52-204, 477-559) so that its known-answer tables still
 * apply; the widths are parameters.  The plan estimate is new: it walks the
 * address stream of the gfx950 kernels in kernels.hip (64 lanes per request,
 * 128-byte lines, 32-byte sectors, 64x64 tiles, row/column packed tables).
 */
#include "model.h"

#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <random>
#include <vector>

namespace cutt {

int glTransactions(const int* seg, int n) {
  if (n <= 0) return 0;
  int count = 1;
  for (int i = 1; i < n; i++) count += (seg[i] != seg[i - 1]);
  return count;
}

int glTransactions(int pos, int n, int accWidth) {
  if (n <= 0) return 0;
  return (pos + n - 1) / accWidth - pos / accWidth + 1;
}

void countCacheLines(const int* seg, int n, int cacheWidth, int& clFull, int& clPart) {
  // Positions increase monotonically, so the lanes that touch one line are a run of equal
  // segment numbers; the line is fully covered when the run has cacheWidth members.
  clFull = clPart = 0;
  int i = 0;
  while (i < n) {
    int j = i + 1;
    while (j < n && seg[j] == seg[i]) j++;
    if (j - i >= cacheWidth)
      clFull++;
    else
      clPart++;
    i = j;
  }
}

void countCacheLines(int pos, int n, int cacheWidth, int& clFull, int& clPart) {
  clFull = clPart = 0;
  if (n <= 0) return;
  const int first = pos / cacheWidth, last = (pos + n - 1) / cacheWidth;
  const bool headPartial = (pos % cacheWidth) != 0;
  const bool tailPartial = ((pos + n) % cacheWidth) != 0;
  if (first == last) {
    if (headPartial || tailPartial) clPart = 1; else clFull = 1;
    return;
  }
  clPart = (int)headPartial + (int)tailPartial;
  clFull = (last - first + 1) - clPart;
}

void countShTransactions(int waveSize, int numBanks, int numThreads, int volMmk, const ShConv* msh,
                         int numMsh, int& sldTran, int& sstTran, int& sldReq, int& sstReq) {
  std::vector<int> perBank(numBanks);
  for (int blockStart = 0; blockStart < volMmk; blockStart += numThreads) {
    const int blockEnd = std::min(volMmk, blockStart + numThreads);
    for (int w0 = blockStart; w0 < blockEnd; w0 += waveSize) {
      const int n = std::min(waveSize, volMmk - w0);
      std::fill(perBank.begin(), perBank.end(), 0);
      int degree = 0;
      for (int l = 0; l < n; l++) {
        const int j = w0 + l;
        int pos = 0;
        for (int k = 0; k < numMsh; k++) pos += ((j / msh[k].c) % msh[k].d) * msh[k].ct;
        degree = std::max(degree, ++perBank[pos % numBanks]);
      }
      sldTran += degree;
      sstTran += 1;
      sldReq += 1;
      sstReq += 1;
    }
  }
}

// ---------------------------------------------------------------------------
namespace {

constexpr int kTile = 64;
constexpr int kLineBytes = 128;
constexpr int kSectorBytes = 32;
constexpr int kLdsBanks = 64;

struct Counts {
  double rdLines = 0, wrLines = 0, rdInstr = 0, wrInstr = 0, wrPartial = 0, rdSectors = 0,
         wrSectors = 0, ldsCycles = 0;
  void add(const Counts& o, double w) {
    rdLines += w * o.rdLines; wrLines += w * o.wrLines; rdInstr += w * o.rdInstr;
    wrInstr += w * o.wrInstr; wrPartial += w * o.wrPartial; rdSectors += w * o.rdSectors;
    wrSectors += w * o.wrSectors; ldsCycles += w * o.ldsCycles;
  }
};

// A contiguous run of n elements at element offset pos: lines, sectors, partial lines.
inline void runCost(int64_t pos, int64_t n, int es, double& lines, double& sectors, double& partial) {
  if (n <= 0) return;
  const int64_t b0 = pos * es, b1 = (pos + n) * es;  // [b0, b1)
  const int64_t l0 = b0 / kLineBytes, l1 = (b1 - 1) / kLineBytes;
  lines += (double)(l1 - l0 + 1);
  sectors += (double)((b1 - 1) / kSectorBytes - b0 / kSectorBytes + 1);
  const bool head = (b0 % kLineBytes) != 0, tail = (b1 % kLineBytes) != 0;
  if (l0 == l1) partial += (head || tail) ? 1 : 0;
  else partial += (int)head + (int)tail;
}

void mbarOffsets(const cuttHipMbar& mb, uint32_t m, int64_t& offIn, int64_t& offOut) {
  offIn = offOut = 0;
  for (int k = 0; k < mb.n; k++) {
    const uint32_t i = m % mb.d[k].extent;
    m /= mb.d[k].extent;
    offIn += (int64_t)i * mb.d[k].strideIn;
    offOut += (int64_t)i * mb.d[k].strideOut;
  }
}

// Offset of row i of a tile axis: i * stride for a single rank, the mixed-radix sum over a fused set.
inline int64_t rowOffset(const cuttHipRowRadix& rr, int64_t stride, int64_t i) {
  if (rr.n == 0) return i * stride;
  int64_t off = 0;
  for (int k = 0; k < rr.n; k++) {
    const int64_t e = rr.extent[k];
    off += (k + 1 < rr.n ? i % e : i) * (int64_t)rr.stride[k];
    i /= e;
  }
  return off;
}

// One tile of w x h elements (w along the input-contiguous axis, h along the Mk axis).
Counts tileCost(bool copy, int es, int64_t offIn, int64_t offOut, int64_t m0, int64_t k0, int w, int h,
                int64_t strideInK, int64_t strideOut, const cuttHipRowRadix& rowsK, const cuttHipRowRadix& rowsM) {
  Counts c;
  double dummy = 0;
  for (int k = 0; k < h; k++) {
    runCost(offIn + m0 + rowOffset(rowsK, strideInK, k0 + k), w, es, c.rdLines, c.rdSectors, dummy);
    c.rdInstr += 1;
  }
  if (copy) {
    for (int k = 0; k < h; k++) {
      runCost(offOut + m0 + (k0 + k) * strideOut, w, es, c.wrLines, c.wrSectors, c.wrPartial);
      c.wrInstr += 1;
    }
  } else {
    for (int m = 0; m < w; m++) {
      runCost(offOut + k0 + rowOffset(rowsM, strideOut, m0 + m), h, es, c.wrLines, c.wrSectors, c.wrPartial);
      c.wrInstr += 1;
    }
    // LDS: one padded-tile write and one read per element row, conflict free.
    c.ldsCycles += (double)(h + w) * (es == 8 ? 4 : 2);
  }
  return c;
}

Counts tiledSample(const Plan& p, bool copy, uint32_t m, std::minstd_rand0& rng, bool everyTile) {
  const int es = p.pb.elemSize;
  const int volMm = copy ? p.tcopy.volMm : p.tiled.volMm;
  const int volMk = copy ? p.tcopy.volMk : p.tiled.volMk;
  const int64_t sIn = copy ? p.tcopy.strideInK : p.tiled.strideInK;
  const int64_t sOut = copy ? p.tcopy.strideOutK : p.tiled.strideOutM;
  static const cuttHipRowRadix kSingle = {};
  const cuttHipRowRadix& rowsK = copy ? kSingle : p.tiled.rowsK;
  const cuttHipRowRadix& rowsM = copy ? kSingle : p.tiled.rowsM;
  int64_t offIn, offOut;
  mbarOffsets(copy ? p.tcopy.mbar : p.tiled.mbar, m, offIn, offOut);
  const int fullM = volMm / kTile, fullK = volMk / kTile;
  const int remM = volMm % kTile, remK = volMk % kTile;
  Counts total;
  if (rowsK.n == 0 && rowsM.n == 0) {
    // equally spaced rows: the full tiles of one Mbar position all cost the same
    if (fullM && fullK)
      total.add(tileCost(copy, es, offIn, offOut, 0, 0, kTile, kTile, sIn, sOut, rowsK, rowsM), (double)fullM * fullK);
    if (remM && fullK)
      total.add(tileCost(copy, es, offIn, offOut, (int64_t)fullM * kTile, 0, remM, kTile, sIn, sOut, rowsK, rowsM), fullK);
    if (remK && fullM)
      total.add(tileCost(copy, es, offIn, offOut, 0, (int64_t)fullK * kTile, kTile, remK, sIn, sOut, rowsK, rowsM), fullM);
    if (remM && remK)
      total.add(tileCost(copy, es, offIn, offOut, (int64_t)fullM * kTile, (int64_t)fullK * kTile, remM, remK,
                         sIn, sOut, rowsK, rowsM), 1);
    return total;
  }
  // Rows over fused ranks start at offsets that differ from tile to tile: a few tiles of every kind
  // (inner, last along Mm, last along Mk, corner) are walked and stand for the others (all of them
  // when the caller asks for the exact count).
  const int tilesM = fullM + (remM ? 1 : 0), tilesK = fullK + (remK ? 1 : 0);
  auto sample = [&](int tmLo, int tmHi, int tkLo, int tkHi) {  // tiles [tmLo, tmHi) x [tkLo, tkHi)
    const int64_t count = (int64_t)(tmHi - tmLo) * (tkHi - tkLo);
    if (count <= 0) return;
    const int64_t n = everyTile ? count : std::min<int64_t>(count, 6);
    for (int64_t i = 0; i < n; i++) {
      int tm, tk;
      if (n == count) {
        tm = tmLo + (int)(i % (tmHi - tmLo));
        tk = tkLo + (int)(i / (tmHi - tmLo));
      } else {
        tm = tmLo + (int)(rng() % (uint32_t)(tmHi - tmLo));
        tk = tkLo + (int)(rng() % (uint32_t)(tkHi - tkLo));
      }
      const int w = std::min(kTile, volMm - tm * kTile), h = std::min(kTile, volMk - tk * kTile);
      total.add(tileCost(copy, es, offIn, offOut, (int64_t)tm * kTile, (int64_t)tk * kTile, w, h, sIn, sOut, rowsK, rowsM),
                (double)count / n);
    }
  };
  sample(0, fullM, 0, fullK);
  sample(fullM, tilesM, 0, fullK);
  sample(0, fullM, fullK, tilesK);
  sample(fullM, tilesM, fullK, tilesK);
  return total;
}

// One staged block of a Packed / PackedSplit plan.
Counts packedSample(const Plan& p, int cls, int64_t offIn, int64_t offOut) {
  const int es = p.pb.elemSize;
  const PackedTables& t = p.tab[cls];
  Counts c;
  std::vector<int64_t> lines, sectors;  // distinct 128-byte lines / 32-byte sectors of one request
  lines.reserve(128);
  sectors.reserve(256);
  // Reads: wavefront requests cover 64 consecutive input-compact positions.
  for (int p0 = 0; p0 < t.vol; p0 += 64) {
    const int p1 = std::min(t.vol, p0 + 64);
    lines.clear();
    sectors.clear();
    int q = p0;
    while (q < p1) {
      const int row = q / t.inCont, col = q % t.inCont;
      const int n = std::min(p1 - q, t.inCont - col);
      const int64_t pos = offIn + t.rowIn[row] + col;
      const int64_t b0 = pos * es, b1 = (pos + n) * es;
      for (int64_t l = b0 / kLineBytes; l <= (b1 - 1) / kLineBytes; l++) lines.push_back(l);
      for (int64_t l = b0 / kSectorBytes; l <= (b1 - 1) / kSectorBytes; l++) sectors.push_back(l);
      q += n;
    }
    std::sort(lines.begin(), lines.end());
    c.rdLines += (double)(std::unique(lines.begin(), lines.end()) - lines.begin());
    std::sort(sectors.begin(), sectors.end());
    c.rdSectors += (double)(std::unique(sectors.begin(), sectors.end()) - sectors.begin());
    c.rdInstr += 1;
  }
  // Writes: 64 consecutive output-compact positions per request.
  std::vector<int> bank(kLdsBanks);
  for (int q0 = 0; q0 < t.vol; q0 += 64) {
    const int q1 = std::min(t.vol, q0 + 64);
    lines.clear();
    sectors.clear();
    int q = q0;
    while (q < q1) {
      const int row = q / t.outCont, col = q % t.outCont;
      const int n = std::min(q1 - q, t.outCont - col);
      const int64_t pos = offOut + t.rowOut[row] + col;
      const int64_t b0 = pos * es, b1 = (pos + n) * es;
      for (int64_t l = b0 / kLineBytes; l <= (b1 - 1) / kLineBytes; l++) lines.push_back(l);
      for (int64_t l = b0 / kSectorBytes; l <= (b1 - 1) / kSectorBytes; l++) sectors.push_back(l);
      q += n;
    }
    std::sort(lines.begin(), lines.end());
    c.wrLines += (double)(std::unique(lines.begin(), lines.end()) - lines.begin());
    std::sort(sectors.begin(), sectors.end());
    c.wrSectors += (double)(std::unique(sectors.begin(), sectors.end()) - sectors.begin());
    c.wrInstr += 1;
    // LDS gather: conflict degree over 4-byte banks; 8-byte words occupy two banks.
    std::fill(bank.begin(), bank.end(), 0);
    int degree = 0;
    const int words = es / 4;
    for (int k = q0; k < q1; k++) degree = std::max(degree, ++bank[(t.shIdx[k] * words) % kLdsBanks]);
    c.ldsCycles += (double)degree * words + words;  // gather read + linear write
  }
  // Partial lines of the output rows (each row is one contiguous run).
  for (size_t r = 0; r < t.rowOut.size(); r++) {
    double l = 0, s = 0;
    runCost(offOut + t.rowOut[r], t.outCont, es, l, s, c.wrPartial);
  }
  return c;
}

}  // namespace

bool estimatePlan(Plan& plan, const cuttHipDeviceProps& props, int numSamples) {
  ModelResult& r = plan.model;
  r = ModelResult();
  const int es = plan.pb.elemSize;
  const double bytes = (double)plan.pb.volume * es;
  if (plan.method == kTrivial) {
    r.rdLines = r.wrLines = bytes / kLineBytes;
    r.rdSectors = r.wrSectors = bytes / kSectorBytes;
    r.usPredicted = 0.0;  // a plain copy always wins (reference src/cuttplan.cpp:705-707)
    return true;
  }
  std::minstd_rand0 rng;  // fixed seed: deterministic plans
  Counts total;
  double tableBytes = 0;
  if (plan.method == kTiled || plan.method == kTiledCopy) {
    const bool copy = plan.method == kTiledCopy;
    const uint32_t volMbar = (uint32_t)plan.split.volMbar;
    const int ns = (numSamples == 0 || (uint32_t)numSamples > volMbar) ? (int)volMbar : numSamples;
    std::uniform_int_distribution<uint32_t> pick(0, volMbar - 1);
    for (int i = 0; i < ns; i++) {
      const uint32_t m = ((uint32_t)ns == volMbar) ? (uint32_t)i : pick(rng);
      total.add(tiledSample(plan, copy, m, rng, numSamples == 0), (double)volMbar / ns);
    }
  } else {
    if (!plan.buildTables()) return false;
    const cuttHipPackedArgs& a = plan.packed;
    const uint32_t ns0 = (uint32_t)a.split[0].numSplit, ns1 = (uint32_t)a.split[1].numSplit;
    const uint32_t items = (uint32_t)a.volMbar * ns0 * ns1;
    const uint32_t numbers = (uint32_t)cuttHipPackedItemNumbers(&a);  // some are empty in item order 1
    const bool all = numSamples == 0 || (uint32_t)numSamples > items;
    const int ns = all ? (int)items : numSamples;
    std::uniform_int_distribution<uint32_t> pick(0, numbers - 1);
    int taken = 0;
    for (uint32_t i = 0; all ? i < numbers : taken < ns; i++) {
      const uint32_t w = all ? i : pick(rng);
      uint32_t s0, s1, m;
      int cls;
      if (!cuttHipDecodeItem(&a, w, &m, &s0, &s1, &cls)) continue;
      taken++;
      const int64_t p0 = (int64_t)s0 * a.split[0].slabFloor + std::min<int64_t>(s0, a.split[0].slabRem);
      const int64_t p1 = (int64_t)s1 * a.split[1].slabFloor + std::min<int64_t>(s1, a.split[1].slabRem);
      int64_t offIn, offOut;
      mbarOffsets(a.mbar, m, offIn, offOut);
      offIn += p0 * a.split[0].strideIn + p1 * a.split[1].strideIn;
      offOut += p0 * a.split[0].strideOut + p1 * a.split[1].strideOut;
      total.add(packedSample(plan, cls, offIn, offOut), (double)items / ns);
    }
    // Every workgroup loads its tables once from L2: 2 bytes per element and 4 per run.
    {
      int big = 0;
      for (int c = 1; c < 4; c++)
        if (plan.tab[c].vol > plan.tab[big].vol) big = c;
      const PackedTables& t = plan.tab[big];
      tableBytes = (double)plan.numBlocks * (2.0 * t.vol + 4.0 * (double)(t.rowIn.size() + t.rowOut.size()));
    }
  }
  r.rdLines = total.rdLines; r.wrLines = total.wrLines;
  r.rdInstr = total.rdInstr; r.wrInstr = total.wrInstr;
  r.wrPartialLines = total.wrPartial;
  r.rdSectors = total.rdSectors; r.wrSectors = total.wrSectors;
  r.ldsCycles = total.ldsCycles;

  // Resident workgroups per CU.
  const double byLds = plan.ldsBytes ? std::floor((double)props.ldsPerCU / (double)plan.ldsBytes) : 32.0;
  // Wavefronts that fit a CU by registers: 512 per SIMD lane, allocated in units of 8, 4 SIMDs.
  double threadsByRegs = (double)props.maxThreadsPerCU;
  if (plan.method == kPacked || plan.method == kPackedSplit) {
    const int regs = cuttHipPackedRegsPerLane(plan.pb.elemSize, plan.packed.elemsPerThread, plan.packed.wideOffsets);
    if (regs > 0) threadsByRegs = std::min(threadsByRegs, 4.0 * 64.0 * std::min(8, 512 / ((regs + 7) / 8 * 8)));
  }
  const double byThreads = std::floor(threadsByRegs / plan.numThreads);
  const double blocksPerCU = std::max(1.0, std::min({byLds, byThreads, 32.0}));
  r.blocksPerCU = blocksPerCU;

  // Distance, in work items, to the item that accesses the next run in memory.
  if (plan.method == kPacked || plan.method == kPackedSplit) {
    const cuttHipPackedArgs& a = plan.packed;
    const Split& sp = plan.split;
    const Problem& pb = plan.pb;
    const double ns0 = a.split[0].numSplit, ns1 = a.split[1].numSplit;
    auto mbarDist = [&](int rank, bool input) -> double {
      double d = ns0 * ns1;
      for (int k = 0; k < a.mbar.n; k++) {
        const bool hit = input ? a.mbar.d[k].strideIn == (uint32_t)pb.strideIn[rank]
                               : a.mbar.d[k].strideOut == (uint32_t)pb.strideOut[rank];
        if (hit && a.mbar.d[k].extent == (uint32_t)pb.dim[rank]) return d;
        d *= a.mbar.d[k].extent;
      }
      return 0.0;
    };
    auto edge = [&](bool input) -> double {
      for (int i = 0; i < pb.rank; i++) {
        const int rk = input ? i : pb.perm[i];
        if (!sp.inMmk[rk]) return mbarDist(rk, input);
        const int slot = sp.method == kPackedSplit ? sp.splitSlot(rk) : -1;
        if (slot >= 0) return slot == 0 ? 1.0 : ns0;
      }
      return 0.0;
    };
    r.rdEdgeDist = edge(true);
    r.wrEdgeDist = edge(false);
  } else if (plan.method == kTiled || plan.method == kTiledCopy) {
    // Distances in workgroups (one tile each).  Along a tiled rank the next run belongs to the next
    // tile: the next workgroup along Mm, superM workgroups on along Mk (strip order).  A rank that
    // fits one tile ends its runs at the rank's end: the next run belongs to another Mbar position.
    const bool copy = plan.method == kTiledCopy;
    const cuttHipMbar& mb = copy ? plan.tcopy.mbar : plan.tiled.mbar;
    const double tilesM = copy ? plan.tcopy.tilesM : plan.tiled.tilesM;
    const double tilesK = copy ? plan.tcopy.tilesK : plan.tiled.tilesK;
    const double superM = copy ? plan.tcopy.superM : plan.tiled.superM;
    const Problem& pb = plan.pb;
    const int order = copy ? plan.tcopy.order : plan.tiled.order;
    auto mbarDist = [&](int rank, bool input) -> double {
      // order 5 walks the Mbar positions strip by strip, the others tensor slice by tensor slice
      double d = order >= 5 ? std::min(superM, tilesM) * tilesK : tilesM * tilesK;
      for (int k = 0; k < mb.n; k++) {
        const bool hit = input ? mb.d[k].strideIn == (uint32_t)pb.strideIn[rank]
                               : mb.d[k].strideOut == (uint32_t)pb.strideOut[rank];
        if (hit && mb.d[k].extent == (uint32_t)pb.dim[rank]) return d;
        d *= mb.d[k].extent;
      }
      return 0.0;
    };
    // input runs lie along rank 0; output runs along the first output rank (Tiled) or rank 0 (TiledCopy)
    // (a Tiled plan over fused rank sets: the runs end where the set ends)
    const int nextIn = copy ? 1 : plan.split.numMm, nextOut = copy ? 1 : plan.split.numMk;
    r.rdEdgeDist = tilesM > 1 ? 1.0 : (nextIn < pb.rank ? mbarDist(nextIn, true) : 0.0);
    if (copy) {
      r.wrEdgeDist = tilesM > 1 ? 1.0 : (pb.rank > 1 ? mbarDist(pb.perm[1], false) : 0.0);
    } else {
      r.wrEdgeDist = tilesK > 1 ? std::min(superM, tilesM) : (nextOut < pb.rank ? mbarDist(pb.perm[nextOut], false) : 0.0);
      // The rank that follows the Mk set in the output may be one of the Mm set (a fused Mm axis): the run
      // next in memory is then the same row of Mk for an Mm index that is `apart` entries on, in another
      // tile along Mm - in the same strip if that is fewer than superM tiles away, else whole strips later
      // (a strip is superM x tilesK tiles, in order 5 for every Mbar position).  Measured on seven 8-byte
      // tensors of the reference's suites whose fused-Mm candidate has one or two tiles along Mk: 1.3-1.55
      // times the estimate that took this distance for zero.
      if (plan.split.numMm > 1 && nextOut < pb.rank && pb.perm[nextOut] > 0 && pb.perm[nextOut] < plan.split.numMm) {
        double apart = 1.0;
        for (int q = 0; q < pb.perm[nextOut]; q++) apart *= pb.dim[q];
        const double tilesApart = apart / kTile;
        double d = 0.0;
        if (tilesApart >= 1.0)
          d = tilesApart < superM ? tilesApart : tilesApart * tilesK * (order >= 5 ? (double)plan.split.volMbar : 1.0);
        if (tilesK > 1) {
          r.wrEdgeOuter = d;
          r.wrOuterShare = 1.0 / tilesK;
        } else {
          r.wrEdgeDist = d;
        }
      }
    }
  }

  // --- time estimate ---
  // The estimate is "time of a same-size device-to-device copy" times an overhead factor that is
  // linear in a few transaction ratios.  The coefficients are a least-squares fit to the measured
  // times of about 7700 candidates over 197 tensors of 1e8-2e8 elements on one MI355X (ranks 2-15, 4-
  // and 8-byte elements, timed by cuttPlanMeasure); over those tensors the plan chosen by this estimate is
  // on average 6 % (median 3.5 %, worst 39 %) slower than the measured best candidate.
  //  - Tiled / TiledCopy: workgroups on one XCD walk neighbouring tiles, so partly used lines are
  //    mostly found in the L2 and extra lines cost less than for the packed kernel; the padding
  //    of edge tiles, whose clamped lanes repeat accesses that hit the L1, costs about a quarter
  //    of a real access.
  //  - Packed / PackedSplit: extra lines on the write side cost about twice as much as on the read
  //    side (partly written lines have to be merged in the L2), and up to three times as much when
  //    the workgroup that writes the rest of the line runs hundreds of work items later (the line
  //    leaves the L2 half written); 4-byte elements cost a little more per byte than 8-byte ones,
  //    and a block cut into slabs a little more than a whole one.
  const double peakBW = (double)props.memClockKHz * 1e3 * 4.0 * (props.memBusWidthBits / 8.0);
  const double tCopy = 2.0 * bytes / (0.64 * peakBW);  // sustained rate of a large D2D copy
  const double lineBytes = bytes / kLineBytes;
  const double rdAmp = r.rdLines / lineBytes, wrAmp = r.wrLines / lineBytes;
  const double partial = r.wrPartialLines / lineBytes;
  // A line shared by two runs is assembled (written) or reused (read) in the L2 only if the other
  // run's workgroup comes soon: "far" rises from 0 when the workgroups in between move one L2's
  // worth of data (4 MB per XCD) to 1 at sixteen times that.
  const double itemBytes = (plan.method == kTiled || plan.method == kTiledCopy)
                               ? 2.0 * kTile * kTile * es
                               : 2.0 * (double)plan.packed.maxVol * es;
  const double l2Bytes = props.l2Bytes > 0 ? (double)props.l2Bytes : 4.0 * 1024 * 1024;
  auto far = [&](double dist) {
    return dist <= 0.0 ? 0.0 : std::min(1.0, std::max(0.0, std::log2(dist * itemBytes / l2Bytes) / 4.0));
  };
  double factor;
  if (plan.method == kTiled || plan.method == kTiledCopy) {
    const bool copy = plan.method == kTiledCopy;
    const double tilesM = copy ? plan.tcopy.tilesM : plan.tiled.tilesM;
    const double tilesK = copy ? plan.tcopy.tilesK : plan.tiled.tilesK;
    // Issued lane-slots over useful ones: a request is 64 lanes wide whatever the tile's width, and
    // an edge tile issues its rows in groups of 16 (loads run over Mk rows; the stores of a Tiled
    // plan run over Mm rows, those of a TiledCopy plan over Mk rows again).
    const double volMm = copy ? plan.tcopy.volMm : plan.tiled.volMm;
    const double volMk = copy ? plan.tcopy.volMk : plan.tiled.volMk;
    auto rows16 = [](double n) { return std::ceil(n / 16.0) * 16.0; };
    const double rdSlots = tilesM * kTile * rows16(volMk);
    const double wrSlots = copy ? rdSlots : rows16(volMm) * tilesK * kTile;
    const double waste = 0.5 * (rdSlots + wrSlots) / (volMm * volMk) - 1.0;
    // Slots of a tile that hold no element cost 4-byte elements half of what they cost 8-byte ones
    // (280 forced plans with a single tile along Mm or Mk: with 0.25 the 4-byte ones ran 0.91 /
    // 0.96 / 1.00 times the prediction at extents 17-32 / 33-48 / 49-64, the 8-byte ones 0.93-0.97
    // whatever the extent; a constant 0.95 for those was tried and only moved single tensors by
    // 25 % in both directions).
    // (Measured on tensors of 0.4-0.9 GB; a tensor that fits the memory-side cache keeps 0.25: with
    // 0.12 a 45 MB tensor with 30-wide tiles was planned Tiled at 58 % of memcpy instead of
    // PackedSplit at 78 %.)
    const double cacheBytes = props.infinityCacheBytes > 0 ? (double)props.infinityCacheBytes : 256.0 * 1024 * 1024;
    const double wasteCost = es == 4 && bytes > cacheBytes ? 0.12 : 0.25;
    factor = (es == 4 ? 1.00 : 0.95) + wasteCost * waste + (es == 4 ? 0.2 : 0.4) * (rdAmp - 1.0) +
             (es == 4 ? 0.1 : 0.2) * (wrAmp - 1.0) + (copy ? (es == 4 ? 0.20 : 0.10) : 0.0) +
             0.7 * partial * ((1.0 - r.wrOuterShare) * far(r.wrEdgeDist) + r.wrOuterShare * far(r.wrEdgeOuter));
    // Tiny slabs of 4-byte elements: with one or two tiles along Mm and exactly two along Mk (a
    // 65..128-long output run cut into a 256-byte piece and a remainder), 46 such plans among 3000
    // random tensors ran 1.29-1.37 times (median) as long as predicted; every other class of tile
    // counts stayed within 6 % of its prediction.
    if (!copy && es == 4 && tilesK == 2.0 && tilesM <= 2.0) factor *= 1.3;
    // ... and whatever the number of tiles along Mm, one or two tiles along Mk (output runs of at
    // most 512 bytes, all of them with partly covered lines at both ends): over the Tiled
    // candidates of 377 random tensors of 4-byte elements that were in reach of the best one, those
    // with one tile along Mk ran 1.10, those with two 1.16 times their estimate.
    else if (!copy && es == 4 && tilesK <= 2.0 && bytes > cacheBytes) factor *= tilesK == 1.0 ? 1.10 : 1.16;
    // The same shape with 8-byte elements: 51 forced plans with two tiles along Mk and one or two
    // along Mm ran 1.11 times as long as predicted in the mean (0.84-1.37), those with three and
    // more tiles along Mm 0.97 times.
    if (!copy && es == 8 && tilesK == 2.0 && tilesM <= 2.0 && bytes > cacheBytes) factor *= 1.1;  // measured at 1.9-3.7 GB
    // A fused Mm axis with one or two tiles along Mk (output runs of at most 1 KB scattered over the rows of
    // several ranks): eleven such 8-byte candidates of the reference's suites ran 0.96-1.35 times this
    // estimate, 1.13 in the mean, and the three that ran 1.2-1.35 times were each picked ahead of a
    // PackedSplit candidate that was 15-25 % faster.
    if (!copy && es == 8 && tilesK <= 2.0 && plan.split.numMm > 1 && bytes > cacheBytes) factor *= 1.15;
    // Workgroups numbered by the address bits their digits move (plan.cpp: addressBitOrder): such plans
    // ran at 0.90-0.93 of this estimate (C2 584 -> 522 us; five 4-byte batched transposes 615 -> 571-597 us),
    // while the aligned PackedSplit candidates they compete with ran 1.1-1.35 times theirs.
    if (!copy && plan.tiled.order == 7) factor *= 0.91;
  } else {
    factor = 1.05 + (es == 4 ? 0.17 : 0.15) * (rdAmp - 1.0) + 0.18 * (wrAmp - 1.0) + 0.08 * partial - (es == 4 ? 0.07 : 0.0) -
             (plan.method == kPacked ? 0.05 : 0.0) + 0.25 * partial * far(r.wrEdgeDist) +
             0.10 * (rdAmp - 1.0) * far(r.rdEdgeDist);
    // Residuals of all candidates in reach of the best one over 600 random tensors and the 80
    // worst 4-byte tensors of the reference's bench 5 (measured / estimated time, regressed on the
    // model's own ratios): what the estimate lacked is the cost of lines that are touched twice
    // when the workgroup with the neighbouring run comes late - the whole excess of lines, not
    // only the partly written ones - and a bump for output runs of 64 bytes to 1 KB.
    // The excess counts lines per request; what a late neighbour can cost is bounded by the lines
    // that two workgroups share (a 4000-byte output run written by 512-byte requests has an excess
    // of 0.21 but shares 0.05 of its lines: (200000,2,500) -> (500,2,200000) with 8-byte elements,
    // cut along the first rank, measured 611-633 us with such runs and 732 us with 64-byte input
    // runs read twice, which the uncapped term ranked the other way round).
    factor += 0.30 * std::min(wrAmp - 1.0, 2.0 * partial) * far(r.wrEdgeDist) +
              (es == 4 ? 0.08 : 0.10) * (rdAmp - 1.0) * far(r.rdEdgeDist);
    {
      const double outBytes = (double)plan.split.volMmkOutCont * es;
      if (outBytes >= 64.0 && outBytes <= 1024.0) factor *= es == 4 ? 1.07 : 1.03;
    }
    // Runs on the 128-byte grid on both sides (no line is requested twice, so the ratios above are all 1 and
    // say nothing about the run lengths): the candidates whose shorter run is 256 bytes ran 5 %, those with
    // 512 bytes and more 10 % faster against their estimates than those with one-line runs (residuals of 2700
    // timed candidates of 112 random tensors with power-of-two extents; with this term the plan picked on those
    // tensors is 4.7 instead of 5.4 % behind the best candidate, on 72 other such tensors of 0.13-2 GB, timed
    // after the term was chosen, 2.3 instead of 4.7 % and 16 instead of 32 % at worst).
    {
      const double cache = props.infinityCacheBytes > 0 ? (double)props.infinityCacheBytes : 256.0 * 1024 * 1024;
      const char* knob = std::getenv("CUTT_MODEL_RUN_LENGTH");  // "0" switches the term off (rule checks)
      if (rdAmp < 1.001 && wrAmp < 1.001 && bytes >= 0.5 * cache && !(knob && knob[0] == '0')) {
        const double shorter = std::min((double)plan.split.volMmkInCont, (double)plan.split.volMmkOutCont) * es;
        factor -= 0.05 * std::min(2.0, std::max(0.0, std::log2(shorter / kLineBytes)));
      }
    }
    // Sixteen elements per lane leave room for one workgroup per CU only; measured about 8 % slower
    // than the counters alone predict.
    if (plan.packed.elemsPerThread > 8) factor += 0.08;
    // Large items run faster than their counters say (fewer barriers and table loads per byte):
    // measured 5-10 % between 4 KB and 64 KB of staged data.
    factor -= 0.10 * (double)plan.ldsBytes / 65536.0;
    // ... and for 4-byte elements most of that comes below 32 KB: over all candidates of 48 random
    // tensors of ranks 4-7 (0.4-0.9 GB) that the model rated within 15 % of its best, items of less
    // than 12 KB ran as predicted, those of 28 KB and more 6-7 % faster than predicted.  Tensors that
    // fit the memory-side cache are another matter (there the few large items of such a plan cost
    // up to 30 %), so the term applies beyond one cache size per buffer only.
    {
      const double cache = props.infinityCacheBytes > 0 ? (double)props.infinityCacheBytes : 256.0 * 1024 * 1024;
      if (es == 4 && bytes > cache) factor -= 0.07 * std::min(1.0, (double)plan.ldsBytes / 32768.0);
    }
    // LDS bank conflicts of the gather, and table reloads when a block has few items.
    factor += 0.5 * r.ldsCycles / ((double)props.cuCount * props.clockKHz * 1e3) / tCopy;
    factor += 0.25 * tableBytes / (2.0 * bytes);
  }
  double t = tCopy * factor;
  // Granularity: with few workgroups per CU the chip fills unevenly and drains slowly.  Measured on
  // tensors of 2M-32M elements the time grows like 1 + (CUs * lanes/1024) / workgroups; for the
  // tens of thousands of workgroups of a large tensor the term vanishes.
  if (plan.numBlocks > 0)
    t *= 1.0 + (double)props.cuCount * ((double)plan.numThreads / 1024.0) / (double)plan.numBlocks;
  if (plan.method == kPacked || plan.method == kPackedSplit) {
    // A workgroup spends about 1.3 us per work item regardless of the item's size (load latency,
    // two barriers, store issue); with small items that, not bandwidth, sets the time:
    // items * 1.3 us spread over the resident workgroups of all CUs.
    const double items = (double)plan.packed.volMbar * plan.packed.split[0].numSplit * plan.packed.split[1].numSplit;
    const double tItems = items * 1.3e-6 / ((double)props.cuCount * blocksPerCU);
    t = std::sqrt(t * t + tItems * tItems);
  }
  r.usPredicted = t * 1e6;
  return true;
}

}  // namespace cutt
