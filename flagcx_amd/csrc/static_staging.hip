// static_staging.hip - the one entry point for callers that may not allocate:
// code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc.  It is flagcxLocalRingReduceScatter (host_staging_ring.cpp) with the
// caller's ring buffer, the ring object, its events and the second stream taken
// away: the nranks-1 peers' slices are staged by one list-copy launch into a
// staging area that is part of the library's own code object (a file-scope
// __device__ array, so every GPU the library runs on holds one copy from the
// moment the code object is loaded there until the process ends), and one reduce
// folds the staged slices and the local slice into recvbuff, in the ring's order
// rank+1, ..., rank (flagcx/service/bootstrap.cc:597-598,651-653).  Both launches
// go to the caller's stream; nothing here calls hipMalloc, hipFree, an event or
// stream constructor, or anything else that allocates.
//
// The array's name is only a host-side handle.  Its device address is looked up
// once per device with hipGetSymbolAddress, with that device current, and only
// that address is ever handed to a launch.
#include "../../include/flagcx_amd.h"
#include "launch.h"

#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>

namespace {

constexpr size_t kStagingBytes = FLAGCX_LOCAL_STATIC_STAGING_BYTES;
constexpr size_t kRegionAlign = 256;

static __device__ __align__(256) unsigned char scratch[kStagingBytes];

constexpr int kMaxDevices = 64;
std::mutex gMutex;
unsigned char *gStaging[kMaxDevices]; // per device: where `scratch` lives there (nullptr: not looked up yet)

// failures go where flagcxLocalGetLastError finds them
flagcxResult_t sfail(flagcxResult_t code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));
flagcxResult_t sfail(flagcxResult_t code, const char *fmt, ...) {
  char text[256];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(text, sizeof(text), fmt, ap);
  va_end(ap);
  flagcx_amd::setLastError(text);
  return code;
}

// The staging area of the current device.  The first call on a device resolves
// the symbol there (the runtime may load the code object at that moment, which is
// why flagcxLocalInit does this ahead of time); later calls only read the table.
flagcxResult_t stagingOfCurrentDevice(unsigned char **out, const char *who) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return sfail(flagcxUnhandledDeviceError, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return sfail(flagcxInternalError, "%s: device %d beyond %d", who, dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(gMutex);
  if (!gStaging[dev]) {
    void *p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      return sfail(flagcxUnhandledDeviceError, "%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
    gStaging[dev] = static_cast<unsigned char *>(p);
  }
  *out = gStaging[dev];
  return flagcxSuccess;
}

inline bool overlap(uintptr_t a, size_t an, uintptr_t b, size_t bn) { return a < b + bn && b < a + an; }

} // namespace

namespace flagcx_amd {

// Called by flagcxLocalInit: looks the staging area up on the current device, so
// that the entry point's first call there finds it (a caller that captures graphs
// calls flagcxLocalInit on each device beforehand).
int resolveStaticStaging() {
  unsigned char *p = nullptr;
  return (int)stagingOfCurrentDevice(&p, "flagcxLocalInit");
}

} // namespace flagcx_amd

#pragma GCC visibility push(default)
extern "C" {

flagcxResult_t flagcxLocalStagedReduceScatterNoAlloc(const void *const *sendbuffs, int nranks, int rank,
                                                     void *recvbuff, size_t recvcount, flagcxDataType_t datatype,
                                                     flagcxRedOp_t op, flagcxStream_t stream) {
  const char *who = "flagcxLocalStagedReduceScatterNoAlloc";
  if (!sendbuffs) return sfail(flagcxInvalidArgument, "%s: sendbuffs is NULL", who);
  if (nranks < 1 || nranks > FLAGCX_LOCAL_MAX_RANKS)
    return sfail(flagcxInvalidArgument, "%s: nranks %d outside [1, %d]", who, nranks, FLAGCX_LOCAL_MAX_RANKS);
  if (rank < 0 || rank >= nranks) return sfail(flagcxInvalidArgument, "%s: rank %d outside [0, %d)", who, rank, nranks);
  int dt, rop;
  memcpy(&dt, &datatype, sizeof(int));
  memcpy(&rop, &op, sizeof(int));
  const size_t ts = (dt >= 0 && dt < (int)flagcxNumTypes) ? flagcxLocalGetDataTypeSize(datatype) : 0;
  if (!ts) return sfail(flagcxInvalidArgument, "%s: unsupported data type %d", who, dt);
  if (rop < 0 || rop >= (int)flagcxNumRedOps)
    return sfail(flagcxInvalidArgument, "%s: unsupported reduction operation %d", who, rop);
  if (recvcount == 0) return flagcxSuccess;
  if (!recvbuff) return sfail(flagcxInvalidArgument, "%s: recvbuff is NULL", who);
  if (recvcount > (kStagingBytes / ts)) // also keeps the products below from wrapping
    return sfail(flagcxInvalidArgument, "%s: %zu elements of %zu bytes exceed the static staging area of %zu bytes",
                 who, recvcount, ts, kStagingBytes);
  const size_t size = recvcount * ts;
  // a peer's region: its slice at recvbuff's position inside a 128-byte cache line (so
  // that the reduce sees the staged inputs and the output at the same position and
  // starts its tiles on their lines), regions 256-byte aligned
  const size_t skew = (uintptr_t)recvbuff & 127u;
  const size_t region = (skew + size + kRegionAlign - 1) / kRegionAlign * kRegionAlign;
  const size_t need = (size_t)(nranks - 1) * region;
  if (need > kStagingBytes)
    return sfail(flagcxInvalidArgument,
                 "%s: %d peers x %zu bytes (regions of %zu) exceed the static staging area of %zu bytes", who,
                 nranks - 1, size, region, kStagingBytes);
  for (int j = 0; j < nranks; j++) {
    if (!sendbuffs[j]) return sfail(flagcxInvalidArgument, "%s: sendbuffs[%d] is NULL", who, j);
    if ((uintptr_t)sendbuffs[j] % ts) return sfail(flagcxInvalidArgument, "%s: sendbuffs[%d] not aligned to %zu", who, j, ts);
    const uintptr_t slice = (uintptr_t)sendbuffs[j] + (size_t)rank * size;
    // in place (flagcx/include/flagcx.h:356) is the local slice itself; any other
    // overlap of the output with a slice that is read is refused
    if (overlap((uintptr_t)recvbuff, size, slice, size) && !(j == rank && slice == (uintptr_t)recvbuff))
      return sfail(flagcxInvalidArgument, "%s: recvbuff overlaps the slice of sendbuffs[%d]", who, j);
  }
  if ((uintptr_t)recvbuff % ts) return sfail(flagcxInvalidArgument, "%s: recvbuff not aligned to %zu", who, ts);
  if (nranks == 1) // nothing to stage (flagcx/service/bootstrap.cc:856-861)
    return flagcxLocalReduceScatter(sendbuffs, 1, 0, recvbuff, recvcount, datatype, op, stream);

  unsigned char *staging = nullptr;
  flagcxResult_t r = stagingOfCurrentDevice(&staging, who);
  if (r != flagcxSuccess) return r;

  // ring order rank+1, ..., rank: the first nranks-1 are the peers, the last is local
  const void *peerSrc[FLAGCX_LOCAL_MAX_RANKS];
  const void *ordered[FLAGCX_LOCAL_MAX_RANKS];
  for (int j = 0; j < nranks - 1; j++) {
    const int peer = (rank + 1 + j) % nranks;
    peerSrc[j] = (const char *)sendbuffs[peer] + (size_t)rank * size;
    ordered[j] = staging + (size_t)j * region + skew;
  }
  ordered[nranks - 1] = (const char *)sendbuffs[rank] + (size_t)rank * size;
  hipStream_t hs = stream ? *reinterpret_cast<hipStream_t *>(stream) : nullptr;
  (void)flagcx_amd::deviceInfo();
  // one launch stages every peer's slice: sources from the list, destinations
  // `region` apart in the staging area
  flagcx_amd::Copy2D c{staging + skew, nullptr, (uint64_t)(nranks - 1), size, 0, region, peerSrc, nullptr, hs};
  const int err = flagcx_amd::launchCopy2D(c);
  if (err) return sfail(flagcxUnhandledDeviceError, "%s: %s", who, hipGetErrorString((hipError_t)err));
  // same stream: the reduce starts when the staging copy has finished
  return flagcxLocalReduce(ordered, nranks, recvbuff, recvcount, datatype, op, stream);
}

} // extern "C"
#pragma GCC visibility pop
