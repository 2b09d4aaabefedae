/*
 * model.h - memory-transaction cost model used by cuttPlan to rank candidates.
 *
 * Counterpart of reference src/cuttGpuModel.h and of cuttPlan_t::countCycles
 * (reference src/cuttplan.cpp:1053-1611): it replays the address stream of a
 * candidate for a few sampled Mbar positions, counts memory transactions, and
 * turns the counts into a time estimate.  Re-derived for gfx950: requests are
 * issued by 64-lane wavefronts, a transaction is one 128-byte line, written
 * lines are tracked at 32-byte sector granularity, LDS has 64 four-byte banks.
 */
#ifndef CUTT_MODEL_H
#define CUTT_MODEL_H

#include <cstdint>

#include "plan.h"

namespace cutt {

// ---- width-parametric counters (same definitions as the reference's) -------
// accWidth / cacheWidth are in elements.

// Transactions of one request whose lanes touch the (sorted) segments seg[0..n).
// Reference src/cuttGpuModel.cpp:52-58.
int glTransactions(const int* seg, int n);
// Transactions of one request that reads n contiguous elements from pos.
// Reference src/cuttGpuModel.cpp:78-85.
int glTransactions(int pos, int n, int accWidth);
// Full and partial cache lines of a monotonically increasing access pattern,
// seg[i] = pos[i] / cacheWidth.  Reference src/cuttGpuModel.cpp:94-116.
void countCacheLines(const int* seg, int n, int cacheWidth, int& clFull, int& clPart);
// Same for n contiguous elements from pos.  Reference src/cuttGpuModel.cpp:187-204.
void countCacheLines(int pos, int n, int cacheWidth, int& clFull, int& clPart);
// LDS transactions of gather reads with per-rank (c, d, ct) strides, bank-conflict degree summed
// over wavefront-sized requests.  Reference src/cuttGpuModel.cpp:477-559.
struct ShConv { int c, d, ct; };
void countShTransactions(int waveSize, int numBanks, int numThreads, int volMmk, const ShConv* msh,
                         int numMsh, int& sldTran, int& sstTran, int& sldReq, int& sstReq);

// ---- plan estimate -----------------------------------------------------------
// Fills plan.model (counters + predicted microseconds).  numSamples = Mbar positions sampled
// (0 = all).  Returns false on internal error.
bool estimatePlan(Plan& plan, const cuttHipDeviceProps& props, int numSamples = 10);

}  // namespace cutt

#endif  // CUTT_MODEL_H
