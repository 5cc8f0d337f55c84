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
  int anyOrder;   // this launch need not wait for the launch before it on the stream to finish (chunks of one call)
  int plusZero;   // op is a sum and the fold also holds members, not listed in src, that are all zeros (kSumZ)
};

// Cached per-process facts about the device the library runs on.
struct DeviceInfo {
  int numCU;
  int ldsPerCU;      // bytes
  bool ldsCaps;      // LDS reservations cap the wavefronts per CU the way ldsReservation assumes
};
const DeviceInfo &deviceInfo();

// Launch shape of a k-input reduce (k = 0: copies) of `tiles` KiB per input: inputs
// whose loads a wavefront keeps in flight (0 = all) and resident one-wave workgroups
// per CU (0 = no cap); the calling thread's flagcxLocalTune* settings applied.
struct LaunchShape {
  int loads, waves;
};
LaunchShape launchShapeFor(int k, uint64_t tiles);
void setWavesPerCU(int k, int waves);
int tunedWavesPerCU(int k); // the explicit setting, or -1
int tunedLoadsInFlight(int k); // the explicit setting (0 = all at once), or -1

// LDS bytes to reserve per workgroup so that at most `waves` one-wave workgroups
// fit on a CU.  0 when no cap is wanted.
int ldsReservation(int waves);

// One launcher per element type; returns a hipError_t value.
typedef int (*ReduceLauncher)(const ReduceCall &);
ReduceLauncher reduceLauncherFor(int dtype);
// n reductions sharing k, op and stream, in as few launches as possible.
typedef int (*ReduceBatchLauncher)(const ReduceCall *, int);
ReduceBatchLauncher reduceBatchLauncherFor(int dtype);

// Host-producer / device-consumer reduce queue (reduce_queue_device.h,
// host_reduce_fifo.cpp).  One entry as the resident consumer kernel reads it.
struct alignas(128) QueueEntry {
  uint64_t src[8];  // inputs in fold order
  uint64_t dst;
  uint64_t nvec;    // 16-byte vectors in the body
  uint32_t head;    // elements before the body
  uint32_t tail;    // elements after it
  uint32_t k;       // number of inputs, 1..8; 0 = stop
  uint32_t flags;   // kQueueFlag*
  uint64_t traffic; // device copy only: (k + 1) * body bytes, written by the consumer's leader
  uint64_t pad[3];
};
static_assert(sizeof(QueueEntry) == 128, "queue entries are 16 words");

// Words of the pinned host header, as in the reference's FIFO
// ([capacity, consumed, produced, ...], flagcx/include/flagcx_kernel.h:75-77),
// plus a state word.
enum : int { kQueueCapacity = 0, kQueueConsumed = 1, kQueueProduced = 2, kQueueState = 3, kQueueHeaderWords = 16 };
// Entry flags: every source shares dst's address modulo 16; the entry reads or
// overwrites what an entry still in flight writes or reads, so it must start after
// everything before it has finished.
enum : uint32_t { kQueueFlagAligned = 1, kQueueFlagAfterAll = 2 };
enum : uint64_t { kQueueIdle = 0, kQueueRunning = 1, kQueueStopped = 2, kQueueTimedOut = 3, kQueueParked = 4 };
// Top bit of the `produced` word: set by the consumer (compare-and-swap against an
// unchanged count) when it leaves an idle queue, seen and cleared by the producer's
// next fetch-and-add, which then launches a new consumer.  One word, so exactly one
// side wins when an entry arrives while the consumer is leaving.
constexpr uint64_t kQueueParkedBit = 1ull << 63;

// Ticket counters of the reduce queue's workers: at most this many, each in a KiB of its own.
constexpr int kQueueMaxTicketCounters = 64;
constexpr int kQueueTicketStride = 128; // 64-bit words

struct QueueKernelArgs {
  uint64_t *hostHeader;          // pinned, device-visible
  const QueueEntry *hostEntries; // pinned ring, `capacity` entries
  QueueEntry *devEntries;        // device copy of the ring the workers read
  uint64_t *devProduced;         // entries forwarded to the device ring; ~0 = abort
  uint32_t *progress;            // per worker: entries finished (low 32 bits)
  uint32_t capacity;
  int64_t maxSpin;
  uint64_t base;                 // entries finished before this launch; device counts are relative to it
  int64_t linger;                // idle polls before the consumer parks; 0 = stay until stopped
  uint64_t windowBytes;          // traffic of the entries the workers may have in work together
  uint64_t *tickets;             // ticket counters, kQueueTicketStride words apart, zero at launch
  uint32_t counters;             // how many of them this launch uses (every one has workers)
  uint32_t drawAhead;            // the queue takes entries of more than four inputs: picks the kernel instantiation
};

// Launches the consumer for one element type: grid = min(occupancy, wavesPerCU) *
// numCU one-wave workgroups, all resident.  Returns a hipError_t value.
typedef int (*ReduceQueueLauncher)(int op, const QueueKernelArgs &, int wavesPerCU, int numCU, int lds,
                                   unsigned maxGrid, hipStream_t, unsigned *grid);
ReduceQueueLauncher reduceQueueLauncherFor(int dtype);
long long asyncMaxSpin(); // async_kernels.hip

// A batch launched before its inputs have arrived (reduce_gate_device.h): its workgroups
// wait until the host's count has passed their descriptor's number.
constexpr int kGateBatchMax = 32; // descriptors per launch, as the plain batch launch
enum : uint64_t { kGateOk = 0, kGateTimedOut = 1 };
struct GateArgs {
  const uint64_t *host; // pinned: descriptors numbered below this count may run
  uint64_t *dev;        // device copy, only ever raised; ~0 = abandoned
  uint64_t *hostState;  // pinned: kGate*
  uint64_t all;         // the launch's leader leaves when the count reaches this
  int64_t maxSpin;
  uint64_t scalarRead;  // dev is uncached device memory: the first read of a wavefront goes through the scalar path
  uint64_t need[kGateBatchMax]; // number of each segment's descriptor
};
// n <= kGateBatchMax reductions that share k (at most 8), op and stream and whose pointers
// agree modulo 16 per reduction; need[i] is the number of calls[i].  hipErrorInvalidValue
// for anything else.
typedef int (*ReduceGatedLauncher)(const ReduceCall *, int n, const GateArgs &);
ReduceGatedLauncher reduceGatedLauncherFor(int dtype);

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
// One source copied to several destinations, up to kFanMaxSeg such copies in one launch: the
// source is read once.  Every destination agrees with its source modulo 16 bytes.
constexpr int kFanMaxDst = 8;
constexpr int kFanMaxSeg = 16;
struct FanoutCall {
  const void *src;
  void *dst[kFanMaxDst];
  int ndst;
  uint64_t bytes;
};
int launchFanout(const FanoutCall *calls, int n, hipStream_t stream);

// Text that flagcxLocalGetLastError returns to the calling thread (c_api.cpp).
void setLastError(const char *text);
// Looks up, for the current device, the library's static staging area
// (static_staging.hip); returns a flagcxResult_t value.
int resolveStaticStaging();

} // namespace flagcx_amd
