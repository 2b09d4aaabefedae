/*
 * tensor_check.hip - kernels behind tensor_check.h (pattern fill, closed-form
 * check, plain copies).  gfx950 only.
 */
#include "tensor_check.h"

#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>

namespace cuttdrv {

#define DRV_HIP(call)                                                                       \
  do {                                                                                      \
    hipError_t e_ = (call);                                                                 \
    if (e_ != hipSuccess) {                                                                 \
      std::fprintf(stderr, "%s:%d HIP error %s\n", __FILE__, __LINE__, hipGetErrorString(e_)); \
      std::exit(2);                                                                         \
    }                                                                                       \
  } while (0)

namespace {

struct CheckGeom {
  int rank;
  unsigned int odim[kMaxCheckRank];            // output extents, fastest first
  unsigned long long istride[kMaxCheckRank];   // input stride of output rank j
};

struct DevResult {
  unsigned long long numWrong, firstPos;
};

__global__ void fillPatternKernel(unsigned int* data, size_t n) {
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) data[i] = (unsigned int)i;
}

__device__ inline unsigned long long expected(unsigned int, unsigned long long idx) { return (unsigned int)idx; }
__device__ inline unsigned long long expected(unsigned long long, unsigned long long idx) {
  unsigned long long lo = (unsigned int)(2 * idx), hi = (unsigned int)(2 * idx + 1);
  return lo | (hi << 32);
}

template <typename T>
__global__ void checkKernel(CheckGeom g, const T* out, unsigned long long vol, DevResult* res) {
  unsigned long long stride = (unsigned long long)gridDim.x * blockDim.x;
  unsigned long long wrong = 0, first = ~0ull;
  for (unsigned long long o = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x; o < vol; o += stride) {
    unsigned long long rest = o, idx = 0;
    for (int j = 0; j < g.rank; j++) {
      unsigned long long q = rest / g.odim[j];
      idx += (rest - q * g.odim[j]) * g.istride[j];
      rest = q;
    }
    if ((unsigned long long)out[o] != expected(T(0), idx)) {
      wrong++;
      if (o < first) first = o;
    }
  }
  if (wrong) {
    atomicAdd(&res->numWrong, wrong);
    atomicMin(&res->firstPos, first);
  }
}

template <typename T>
__global__ void copyPerLaneKernel(const T* in, T* out, size_t n) {
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = in[i];
}

__global__ void copyVector16Kernel(const uint4* in, uint4* out, size_t n) {
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) out[i] = in[i];
}

__global__ void copySmallBlocksKernel(const uint4* in, uint4* out, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = in[i];
}

__global__ void copyTailKernel(const unsigned char* in, unsigned char* out, size_t from, size_t bytes) {
  size_t i = from + threadIdx.x;
  if (i < bytes) out[i] = in[i];
}

int gridFor(size_t n, int threads) {
  size_t blocks = (n + threads - 1) / threads;
  size_t cap = 256 * 16;  // 16 workgroups per CU keep a grid-stride loop busy
  return (int)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

}  // namespace

TensorChecker::TensorChecker() { DRV_HIP(hipMalloc(&dResult_, sizeof(DevResult))); }

TensorChecker::~TensorChecker() {
  if (dResult_) (void)hipFree(dResult_);
}

void TensorChecker::fillPattern(void* data, size_t numWords) {
  fillPatternKernel<<<gridFor(numWords, 256), 256>>>((unsigned int*)data, numWords);
  DRV_HIP(hipGetLastError());
  DRV_HIP(hipDeviceSynchronize());
}

void TensorChecker::fillBytes(void* data, int value, size_t bytes) {
  DRV_HIP(hipMemsetAsync(data, value, bytes, 0));
}

CheckResult TensorChecker::check(int rank, const int* dim, const int* permutation, size_t elemSize,
                                 const void* out) {
  CheckResult r;
  if (rank < 1 || rank > kMaxCheckRank || (elemSize != 4 && elemSize != 8)) {
    r.numWrong = ~0ull;
    return r;
  }
  CheckGeom g;
  g.rank = rank;
  unsigned long long istrideOfInput[kMaxCheckRank];
  unsigned long long vol = 1;
  for (int i = 0; i < rank; i++) {
    istrideOfInput[i] = vol;
    vol *= (unsigned long long)dim[i];
  }
  for (int j = 0; j < rank; j++) {
    g.odim[j] = (unsigned int)dim[permutation[j]];
    g.istride[j] = istrideOfInput[permutation[j]];
  }
  DevResult init = {0ull, ~0ull};
  DRV_HIP(hipMemcpy(dResult_, &init, sizeof(init), hipMemcpyHostToDevice));
  int grid = gridFor(vol, 256);
  if (elemSize == 4)
    checkKernel<unsigned int><<<grid, 256>>>(g, (const unsigned int*)out, vol, (DevResult*)dResult_);
  else
    checkKernel<unsigned long long><<<grid, 256>>>(g, (const unsigned long long*)out, vol, (DevResult*)dResult_);
  DRV_HIP(hipGetLastError());
  DevResult dr;
  DRV_HIP(hipMemcpy(&dr, dResult_, sizeof(dr), hipMemcpyDeviceToHost));
  r.numWrong = dr.numWrong;
  if (dr.numWrong) {
    r.firstPos = dr.firstPos;
    unsigned long long rest = dr.firstPos, idx = 0;
    for (int j = 0; j < rank; j++) {
      idx += (rest % g.odim[j]) * g.istride[j];
      rest /= g.odim[j];
    }
    unsigned long long got = 0;
    DRV_HIP(hipMemcpy(&got, (const char*)out + dr.firstPos * elemSize, elemSize, hipMemcpyDeviceToHost));
    r.got = got;
    r.want = elemSize == 4 ? (unsigned int)idx
                           : ((unsigned long long)(unsigned int)(2 * idx) | ((unsigned long long)(unsigned int)(2 * idx + 1) << 32));
  }
  return r;
}

bool TensorChecker::checkAndReport(int rank, const int* dim, const int* permutation, size_t elemSize,
                                   const void* out) {
  CheckResult r = check(rank, dim, permutation, elemSize, out);
  if (r.numWrong == 0) return true;
  std::printf("check FAILED: %llu wrong elements, first at output position %llu: got 0x%llx, expected 0x%llx\n",
              r.numWrong, r.firstPos, r.got, r.want);
  return false;
}

void copyPerLane(const void* in, void* out, size_t bytes, size_t elemSize, void* stream) {
  size_t n = bytes / elemSize;
  hipStream_t s = (hipStream_t)stream;
  if (elemSize == 4)
    copyPerLaneKernel<unsigned int><<<gridFor(n, 256), 256, 0, s>>>((const unsigned int*)in, (unsigned int*)out, n);
  else
    copyPerLaneKernel<unsigned long long><<<gridFor(n, 256), 256, 0, s>>>((const unsigned long long*)in, (unsigned long long*)out, n);
  DRV_HIP(hipGetLastError());
}

void copyVector16(const void* in, void* out, size_t bytes, void* stream) {
  size_t n = bytes / 16;
  hipStream_t s = (hipStream_t)stream;
  if (n) copyVector16Kernel<<<gridFor(n, 256), 256, 0, s>>>((const uint4*)in, (uint4*)out, n);
  if (bytes % 16) copyTailKernel<<<1, 64, 0, s>>>((const unsigned char*)in, (unsigned char*)out, n * 16, bytes);
  DRV_HIP(hipGetLastError());
}

void copySmallBlocks(const void* in, void* out, size_t bytes, void* stream) {
  size_t n = bytes / 16;
  hipStream_t s = (hipStream_t)stream;
  size_t blocks = (n + 255) / 256;
  if (blocks > 0x7fffffffull) {
    std::fprintf(stderr, "copySmallBlocks: %zu bytes need too many workgroups\n", bytes);
    std::exit(2);
  }
  if (n) copySmallBlocksKernel<<<(int)blocks, 256, 0, s>>>((const uint4*)in, (uint4*)out, n);
  if (bytes % 16) copyTailKernel<<<1, 64, 0, s>>>((const unsigned char*)in, (unsigned char*)out, n * 16, bytes);
  DRV_HIP(hipGetLastError());
}

}  // namespace cuttdrv
