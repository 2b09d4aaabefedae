/*
 * hip_layer.hip - HIP runtime side of the C-ABI layer declared in hip_layer.h:
 * device queries, allocation, copies, memset, events.  No device code here (the layer's plain
 * arithmetic is in layer_math.cpp).
 *
 * Unlike the reference's helpers (reference src/CudaUtils.h:35-42 prints and
 * calls exit(1) on any runtime error) every function reports the error code
 * to its caller, which turns it into CUTT_INTERNAL_ERROR.
 */
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstring>

#include "hip_layer.h"

static std::atomic<unsigned long long> gMallocCalls{0}, gUploadCalls{0};

extern "C" int cuttHipGetDevice(int* device) { return (int)hipGetDevice(device); }

extern "C" int cuttHipGetDeviceProps(int device, cuttHipDeviceProps* p) {
  if (!p) return (int)hipErrorInvalidValue;
  hipDeviceProp_t d;
  hipError_t e = hipGetDeviceProperties(&d, device);
  if (e != hipSuccess) return (int)e;
  std::memset(p, 0, sizeof(*p));
  p->cuCount = d.multiProcessorCount;
  p->waveSize = d.warpSize;
  p->maxThreadsPerBlock = d.maxThreadsPerBlock;
  p->maxThreadsPerCU = d.maxThreadsPerMultiProcessor;
  p->ldsPerBlock = d.sharedMemPerBlock;
  p->ldsPerCU = d.maxSharedMemoryPerMultiProcessor;
  p->clockKHz = d.clockRate;
  p->memClockKHz = d.memoryClockRate;
  p->memBusWidthBits = d.memoryBusWidth;
  p->l2Bytes = d.l2CacheSize;
  p->maxGridX = d.maxGridSize[0];
  std::strncpy(p->arch, d.gcnArchName, sizeof(p->arch) - 1);
  // The runtime does not report the memory-side cache; MI300X and MI355X have 256 MB.
  if (std::strncmp(p->arch, "gfx94", 5) == 0 || std::strncmp(p->arch, "gfx95", 5) == 0)
    p->infinityCacheBytes = (size_t)256 << 20;
  return 0;
}

extern "C" int cuttHipMalloc(void** ptr, size_t bytes) {
  gMallocCalls++;
  return (int)hipMalloc(ptr, bytes);
}
extern "C" void cuttHipCallCounts(unsigned long long* mallocs, unsigned long long* uploads) {
  if (mallocs) *mallocs = gMallocCalls;
  if (uploads) *uploads = gUploadCalls;
}
extern "C" int cuttHipFree(void* ptr) { return (int)hipFree(ptr); }

extern "C" int cuttHipMemcpyHtoD(void* dst, const void* src, size_t bytes) {
  gUploadCalls++;
  return (int)hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice);
}

extern "C" int cuttHipMemcpyDtoDAsync(void* dst, const void* src, size_t bytes, void* stream) {
  return (int)hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, (hipStream_t)stream);
}

extern "C" int cuttHipMemsetAsync(void* dst, int value, size_t bytes, void* stream) {
  return (int)hipMemsetAsync(dst, value, bytes, (hipStream_t)stream);
}

extern "C" int cuttHipDeviceSynchronize(void) { return (int)hipDeviceSynchronize(); }

extern "C" int cuttHipEventCreate(void** event) {
  hipEvent_t e;
  hipError_t r = hipEventCreate(&e);
  if (r == hipSuccess) *event = (void*)e;
  return (int)r;
}
extern "C" int cuttHipEventDestroy(void* event) { return (int)hipEventDestroy((hipEvent_t)event); }
extern "C" int cuttHipEventRecord(void* event, void* stream) {
  return (int)hipEventRecord((hipEvent_t)event, (hipStream_t)stream);
}
extern "C" int cuttHipEventSynchronize(void* event) { return (int)hipEventSynchronize((hipEvent_t)event); }
extern "C" int cuttHipEventElapsedMs(void* start, void* stop, float* ms) {
  return (int)hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop);
}
extern "C" const char* cuttHipErrorString(int err) { return hipGetErrorString((hipError_t)err); }
