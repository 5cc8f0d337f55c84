// launch.h - host-side plumbing shared by the kernel translation units and the
// C ABI layer.  Nothing here is exported.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace flagcx_amd {

constexpr int kMaxRanks = 64;

// What the C ABI hands to a typed reduce launcher after validation.
struct ReduceCall {
  const void *src[kMaxRanks];
  void *dst;
  uint64_t count; // elements
  int k;
  int op;         // flagcxRedOp_t value
  hipStream_t stream;
};

// Cached per-process facts about the device the library runs on.
struct DeviceInfo {
  int numCU;
  int ldsPerCU; // bytes
};
const DeviceInfo &deviceInfo();

// Resident single-wave workgroups per CU for a k-input reduce (k = 0: copies).
int wavesPerCUFor(int k);
void setWavesPerCU(int k, int waves);

// LDS bytes to reserve per workgroup so that at most `waves` one-wave workgroups
// fit on a CU.  0 when no cap is wanted.
int ldsReservation(int waves);

// One launcher per element type; returns a hipError_t value.
typedef int (*ReduceLauncher)(const ReduceCall &);
ReduceLauncher reduceLauncherFor(int dtype);
// n reductions sharing k, op and stream, in as few launches as possible.
typedef int (*ReduceBatchLauncher)(const ReduceCall *, int);
ReduceBatchLauncher reduceBatchLauncherFor(int dtype);

// Byte movers (copy_kernels.hip); all return a hipError_t value.
struct Copy2D {
  void *dst;
  const void *src;
  uint64_t nchunks, chunkBytes, srcStride, dstStride;
  const void *const *srcList; // host arrays, or NULL
  void *const *dstList;
  hipStream_t stream;
};
int launchCopy2D(const Copy2D &c);
int launchFill(void *p0, uint64_t n0, void *p1, uint64_t n1, int value, hipStream_t stream);

} // namespace flagcx_amd
