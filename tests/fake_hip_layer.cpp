// A stand-in for the runtime half of the library's internal C-ABI layer (cutt_amd/csrc/hip_layer.h),
// for host-only tests of the plan API: "device" memory is host memory, a "launch" reads every word
// of the plan's index tables (so that a sanitizer sees a plan freed under a running cuttExecute)
// and takes a little time, events and synchronisation do nothing.  The layer's arithmetic
// (division constants, Mbar tables) is the library's own layer_math.cpp.
// CUTT_FAKE_ZERO_PROPS=1 reports a device whose clock, bus width, CU count and L2 size read zero.
#include <atomic>
#include <chrono>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <thread>
#include <vector>

#include "hip_layer.h"

namespace cutt {
cuttHipDeviceProps defaultMI355XProps();
}

static std::atomic<uint64_t> gSink;
static std::atomic<unsigned long long> gMallocCalls{0}, gUploadCalls{0};
// The index tables of the most recent packed "launch", class by class: rowIn, rowOut, shIdx.
static std::vector<uint32_t> gLastTables;
static std::mutex gLastTablesLock;

static void touch(const cuttHipPackedArgs* a) {
  uint64_t sum = 0;
  for (int c = 0; c < 4; c++) {
    if (((c & 1) && a->split[0].slabRem == 0) || ((c & 2) && a->split[1].slabRem == 0)) continue;
    const cuttHipPackedClass& k = a->cls[c];
    for (int i = 0; i < k.vol / k.inCont; i++) sum += k.rowIn[i];
    for (int i = 0; i < k.vol / k.outCont; i++) sum += k.rowOut[i];
    for (int i = 0; i < k.vol; i++) sum += k.shIdx[i];
  }
  gSink = sum;
  {
    std::lock_guard<std::mutex> guard(gLastTablesLock);
    gLastTables.clear();
    for (int c = 0; c < 4; c++) {
      if (((c & 1) && a->split[0].slabRem == 0) || ((c & 2) && a->split[1].slabRem == 0)) continue;
      const cuttHipPackedClass& k = a->cls[c];
      gLastTables.insert(gLastTables.end(), k.rowIn, k.rowIn + k.vol / k.inCont);
      gLastTables.insert(gLastTables.end(), k.rowOut, k.rowOut + k.vol / k.outCont);
      gLastTables.insert(gLastTables.end(), k.shIdx, k.shIdx + k.vol);
    }
  }
  std::this_thread::sleep_for(std::chrono::microseconds(50));
}

extern "C" {
int cuttHipGetDevice(int* device) { *device = 0; return 0; }
int cuttHipGetDeviceProps(int, cuttHipDeviceProps* p) {
  *p = cutt::defaultMI355XProps();
  const char* z = std::getenv("CUTT_FAKE_ZERO_PROPS");
  if (z && std::atoi(z)) p->memClockKHz = p->memBusWidthBits = p->cuCount = p->l2Bytes = p->clockKHz = 0;
  return 0;
}
int cuttHipMalloc(void** ptr, size_t bytes) { gMallocCalls++; *ptr = std::malloc(bytes ? bytes : 1); return *ptr ? 0 : 2; }
void cuttHipCallCounts(unsigned long long* mallocs, unsigned long long* uploads) {
  if (mallocs) *mallocs = gMallocCalls;
  if (uploads) *uploads = gUploadCalls;
}
// (test hook of this stand-in only) copies the tables of the most recent packed launch; returns their length
size_t fakeLastPackedTables(uint32_t* out, size_t capacity) {
  std::lock_guard<std::mutex> guard(gLastTablesLock);
  for (size_t i = 0; i < gLastTables.size() && i < capacity; i++) out[i] = gLastTables[i];
  return gLastTables.size();
}
int cuttHipFree(void* ptr) { std::free(ptr); return 0; }
int cuttHipMemcpyHtoD(void* dst, const void* src, size_t bytes) { gUploadCalls++; std::memcpy(dst, src, bytes); return 0; }
int cuttHipMemcpyDtoDAsync(void* dst, const void* src, size_t bytes, void*) { std::memcpy(dst, src, bytes); return 0; }
int cuttHipMemsetAsync(void* dst, int value, size_t bytes, void*) { std::memset(dst, value, bytes); return 0; }
int cuttHipDeviceSynchronize(void) { return 0; }
int cuttHipEventCreate(void** event) { *event = std::malloc(1); return 0; }
int cuttHipEventDestroy(void* event) { std::free(event); return 0; }
int cuttHipEventRecord(void*, void*) { return 0; }
int cuttHipEventSynchronize(void*) { return 0; }
int cuttHipEventElapsedMs(void*, void*, float* ms) { *ms = 1.0f; return 0; }
const char* cuttHipErrorString(int) { return "fake layer"; }
int cuttHipValidateTiled(const cuttHipTiledArgs* a) { return a ? 0 : 1; }
int cuttHipValidateTiledCopy(const cuttHipTiledCopyArgs* a) { return a ? 0 : 1; }
int cuttHipValidatePacked(const cuttHipPackedArgs* a) { return a ? 0 : 1; }
int cuttHipLaunchTiled(const cuttHipTiledArgs*, const void*, void*, void*) { return 0; }
int cuttHipLaunchTiledCopy(const cuttHipTiledCopyArgs*, const void*, void*, void*) { return 0; }
int cuttHipLaunchPacked(const cuttHipPackedArgs* a, const void*, void*, void*) { touch(a); return 0; }
int cuttHipLaunchCopy(const void*, void*, size_t, int, void*) { return 0; }
int cuttHipPreparePacked(void) { return 0; }
int cuttHipCountTiled(const cuttHipTiledArgs*, cuttHipStreamCounts*, void*) { return 1; }
int cuttHipCountTiledCopy(const cuttHipTiledCopyArgs*, cuttHipStreamCounts*, void*) { return 1; }
int cuttHipCountPacked(const cuttHipPackedArgs*, cuttHipStreamCounts*, void*) { return 1; }
int cuttHipScratch(void** ptr, size_t* bytes) {
  static unsigned char scratch[CUTT_HIP_SCRATCH_BYTES];
  *ptr = scratch;
  *bytes = sizeof(scratch);
  return 0;
}
int cuttHipLaunchTableBuild(const cuttHipTableBuildArgs* a, void*) {
  auto radix = [](const cuttHipRadixList& l, uint32_t i) {
    uint32_t off = 0;
    for (int k = 0; k < l.n; k++) {
      off += (i % l.extent[k]) * l.stride[k];
      i /= l.extent[k];
    }
    return off;
  };
  for (uint32_t i = 0; i < a->count[0]; i++) a->rowIn[i] = radix(a->list[0], i);
  for (uint32_t i = 0; i < a->count[1]; i++) a->rowOut[i] = radix(a->list[1], i);
  for (uint32_t i = 0; i < a->count[2]; i++) {
    const uint32_t pos = radix(a->list[2], i);
    a->shIdx[i] = (uint16_t)(pos + (pos >> a->padShift));
  }
  return 0;
}
int cuttHipPackedRegsPerLaneLoaded(int, int, int) { return -1; }
}
