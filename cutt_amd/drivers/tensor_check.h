/*
 * tensor_check.h - device-side input pattern and closed-form result check for
 * the native test and benchmark drivers.
 *
 * Plays the part of the reference's TensorTester (src/TensorTester.h:31-60,
 * src/TensorTester.cu:33-218): the input buffer holds 32-bit word i = i, so a
 * 4-byte element e reads as e and an 8-byte element e as the word pair
 * (2e, 2e+1); after a transpose, output element o must hold the input element
 * whose linear index follows from o's coordinates in the permuted tensor.
 * The check runs on the GPU, so full-size tensors are verified in
 * milliseconds, and it uses nothing of the library under test.
 */
#ifndef CUTT_DRIVERS_TENSOR_CHECK_H
#define CUTT_DRIVERS_TENSOR_CHECK_H

#include <cstddef>
#include <cstdint>

namespace cuttdrv {

const int kMaxCheckRank = 32;

struct CheckResult {
  unsigned long long numWrong = 0;   // output elements that differ from the closed form
  unsigned long long firstPos = 0;   // smallest wrong output position (valid if numWrong > 0)
  unsigned long long got = 0, want = 0;
};

class TensorChecker {
 public:
  TensorChecker();
  ~TensorChecker();
  TensorChecker(const TensorChecker&) = delete;
  TensorChecker& operator=(const TensorChecker&) = delete;

  // data[i] = i for i < numWords (32-bit words)
  void fillPattern(void* data, size_t numWords);
  // every byte of data[0, bytes) = value
  void fillBytes(void* data, int value, size_t bytes);
  // Compare `out` (elemSize 4 or 8) with the transpose of the pattern; synchronises.
  // rank 1 with permutation {0} checks a plain copy.
  CheckResult check(int rank, const int* dim, const int* permutation, size_t elemSize, const void* out);
  // Same, and prints the first difference; returns true if the output is right.
  bool checkAndReport(int rank, const int* dim, const int* permutation, size_t elemSize, const void* out);

 private:
  void* dResult_ = nullptr;
};

// Plain device-to-device copy kernels for the memory-copy benchmark (counterparts of the
// reference's scalarCopy / vectorCopy / memcpyFloat, src/CudaMemcpy.cu:33-145).  Asynchronous on
// `stream`.
void copyPerLane(const void* in, void* out, size_t bytes, size_t elemSize, void* stream);   // one element per lane and step
void copyVector16(const void* in, void* out, size_t bytes, void* stream);                   // 16 bytes per lane and step
void copySmallBlocks(const void* in, void* out, size_t bytes, void* stream);                // 16 bytes per lane, one step per workgroup

}  // namespace cuttdrv

#endif
