// host_reduce_fifo.cpp - host side of the host-producer / device-consumer reduce
// queue: the pair `enqueue(flagcxReduceTrigger)` / device `dequeue` that the
// reference declares and leaves commented out
// (flagcx/include/flagcx_kernel.h:52-73,96-98).  Allocation mirrors
// flagcxFifo::flagcxFifoInit (flagcx/core/flagcx_kernel_host.cc:31-45): a pinned,
// device-mapped buffer of 64-bit words [capacity, consumed, produced, ...] followed
// by the entries; the consumer is one resident kernel on a stream the queue owns
// (reduce_queue_device.h), the way the kernel proxy owns a dedicated stream
// (flagcx/core/proxy.cc:1094-1097).
//
// A queue is typed (element type, op) when it is created: a collective has one
// type and one op, and the consumer kernel is compiled per pair.  Entries carry
// 1..8 inputs; the host validates every entry and splits it into head / 16-byte
// body / tail before the device sees it.
#include "../../include/flagcx_amd.h"
#include "launch.h"

#include <sched.h>

#include <atomic>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <mutex>
#include <new>

using namespace flagcx_amd;

struct flagcxLocalReduceFifo {
  uint64_t *header = nullptr;       // pinned: kQueueHeaderWords words, then the entry ring
  QueueEntry *hostEntries = nullptr;
  void *devBlock = nullptr;         // device ring | devProduced | progress words | ticket counters
  QueueEntry *devEntries = nullptr;
  uint64_t *devProduced = nullptr;
  uint32_t *progress = nullptr;
  uint64_t *tickets = nullptr;
  uint32_t capacity = 0;
  unsigned maxGrid = 0;
  unsigned grid = 0;
  int maxRanks = 0, dtype = 0, op = 0;
  int wavesPerCU = 8;               // resident one-wave workgroups per CU
  size_t typeSize = 0;
  hipStream_t stream = nullptr;
  uint64_t produced = 0;            // host copy of header[kQueueProduced]
  uint64_t lastAfterAll = 0;        // index of the youngest entry marked kQueueFlagAfterAll
  bool started = false;             // between Start and Stop
  bool stopSent = false;
  uint64_t windowBytes = 256ull << 20; // traffic of the entries in work together
  int64_t linger = 64;              // idle polls of the leader before the consumer parks (0: never)
  std::mutex mu;                    // producers may be several threads
  char lastError[256] = "";
};

namespace {

flagcxResult_t qfail(flagcxLocalReduceFifo *q, flagcxResult_t code, const char *fmt, ...)
    __attribute__((format(printf, 3, 4)));
flagcxResult_t qfail(flagcxLocalReduceFifo *q, flagcxResult_t code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  if (q) vsnprintf(q->lastError, sizeof(q->lastError), fmt, ap);
  va_end(ap);
  return code;
}

inline uint64_t headerLoad(const flagcxLocalReduceFifo *q, int word) {
  return __atomic_load_n(q->header + word, __ATOMIC_ACQUIRE);
}

inline uint64_t producedLoad(const flagcxLocalReduceFifo *q) {
  return headerLoad(q, kQueueProduced) & ~kQueueParkedBit;
}

inline bool alive(uint64_t state) { return state == kQueueRunning || state == kQueueParked; }

inline bool overlaps(uintptr_t x, uintptr_t y, uint64_t xbytes, uint64_t ybytes) {
  return x < y + ybytes && y < x + xbytes;
}

// Launches a consumer that takes over at entry `base` (everything before it is
// finished).  The caller holds the mutex.
flagcxResult_t launchConsumer(flagcxLocalReduceFifo *q, uint64_t base, const char *who) {
  __atomic_store_n(q->header + kQueueState, (uint64_t)kQueueRunning, __ATOMIC_RELEASE);
  const size_t clearBytes = 128 + (size_t)q->maxGrid * sizeof(uint64_t) +
                            (size_t)kQueueMaxTicketCounters * kQueueTicketStride * sizeof(uint64_t);
  hipError_t e = hipMemsetAsync(q->devProduced, 0, clearBytes, q->stream);
  if (e != hipSuccess) return qfail(q, flagcxUnhandledDeviceError, "%s: %s", who, hipGetErrorString(e));
  QueueKernelArgs a;
  a.hostHeader = q->header;
  a.hostEntries = q->hostEntries;
  a.devEntries = q->devEntries;
  a.devProduced = q->devProduced;
  a.progress = q->progress;
  a.capacity = q->capacity;
  a.maxSpin = asyncMaxSpin();
  a.base = base;
  a.linger = q->linger;
  a.windowBytes = q->windowBytes;
  a.tickets = q->tickets;
  a.counters = 1; // the launcher sets it from the grid
  a.drawAhead = q->maxRanks > 4 ? 1u : 0u;
  // LDS is reserved only to spread the resident wavefronts over the CUs (at most
  // `waves` + 2 fit on one), in whole 1280-byte allocation granules.  A fifth of
  // every CU's LDS stays free, so that other launches that need LDS (this library's
  // own reductions on other streams) still make progress next to the consumer.
  const int waves = q->wavesPerCU;
  const int lds = ((deviceInfo().ldsPerCU - 32 * 1024) / waves) / 1280 * 1280;
  const int err = reduceQueueLauncherFor(q->dtype)(q->op, a, waves, deviceInfo().numCU, lds, q->maxGrid, q->stream,
                                                   &q->grid);
  if (err) {
    __atomic_store_n(q->header + kQueueState, (uint64_t)kQueueIdle, __ATOMIC_RELEASE);
    return qfail(q, flagcxUnhandledDeviceError, "%s: %s", who, hipGetErrorString((hipError_t)err));
  }
  return flagcxSuccess;
}

// Publishes the entry already written at index q->produced.  If the consumer had
// parked (the bit comes back with the old count), the bit is cleared and a new
// consumer is launched from this entry on.  The caller holds the mutex.
flagcxResult_t publishEntry(flagcxLocalReduceFifo *q, const char *who, bool *wasParked) {
  const uint64_t old = __atomic_fetch_add(q->header + kQueueProduced, 1, __ATOMIC_ACQ_REL);
  q->produced++;
  *wasParked = (old & kQueueParkedBit) != 0;
  if (!*wasParked) return flagcxSuccess;
  __atomic_fetch_and(q->header + kQueueProduced, ~kQueueParkedBit, __ATOMIC_ACQ_REL);
  return flagcxSuccess;
}

// Appends one validated entry; the caller holds the mutex.
flagcxResult_t appendEntry(flagcxLocalReduceFifo *q, const QueueEntry &in, uint64_t *ticket, const char *who) {
  if (!q->started || q->stopSent) return qfail(q, flagcxInvalidUsage, "%s: the queue is not running", who);
  const uint64_t state = headerLoad(q, kQueueState);
  if (!alive(state))
    return qfail(q, flagcxInternalError, "%s: the consumer has exited (state %lld)", who, (long long)state);
  const uint64_t consumed = headerLoad(q, kQueueConsumed);
  if (q->produced - consumed >= q->capacity) return flagcxInProgress; // full: retry
  // Entries are folded concurrently.  One that reads or overwrites what an entry
  // still in flight writes, or overwrites what it reads, is marked to start after
  // everything before it; entries older than the last such mark are finished by
  // the time anything behind the mark starts, so only younger ones are compared.
  QueueEntry e = in;
  const size_t ts = q->typeSize;
  auto bytesOf = [ts](const QueueEntry &x) { return ((uint64_t)x.head + x.tail) * ts + x.nvec * 16; };
  const uint64_t eb = bytesOf(e);
  for (uint64_t j = consumed > q->lastAfterAll ? consumed : q->lastAfterAll; j < q->produced; j++) {
    const QueueEntry &o = q->hostEntries[j % q->capacity];
    const uint64_t ob = bytesOf(o);
    bool hit = overlaps((uintptr_t)e.dst, (uintptr_t)o.dst, eb, ob);
    for (uint32_t a = 0; !hit && a < e.k; a++) hit = overlaps((uintptr_t)e.src[a], (uintptr_t)o.dst, eb, ob);
    for (uint32_t a = 0; !hit && a < o.k; a++) hit = overlaps((uintptr_t)e.dst, (uintptr_t)o.src[a], eb, ob);
    if (hit) {
      e.flags |= kQueueFlagAfterAll;
      q->lastAfterAll = q->produced;
      break;
    }
  }
  memcpy(q->hostEntries + q->produced % q->capacity, &e, sizeof(e));
  const uint64_t index = q->produced;
  bool wasParked;
  flagcxResult_t r = publishEntry(q, who, &wasParked);
  if (r == flagcxSuccess && wasParked) r = launchConsumer(q, index, who);
  if (ticket) *ticket = q->produced;
  return r;
}

flagcxResult_t buildEntry(flagcxLocalReduceFifo *q, const void *const *srcs, int k, void *dst, uint64_t count,
                          QueueEntry &e, bool *empty, const char *who) {
  *empty = true;
  if (k < 1 || k > q->maxRanks) return qfail(q, flagcxInvalidArgument, "%s: nranks %d outside [1, %d]", who, k, q->maxRanks);
  if (count == 0) return flagcxSuccess;
  const size_t ts = q->typeSize;
  if (!dst) return qfail(q, flagcxInvalidArgument, "%s: recvbuff is NULL", who);
  if ((uintptr_t)dst % ts) return qfail(q, flagcxInvalidArgument, "%s: recvbuff not aligned to its element size", who);
  if (count > UINT64_MAX / ts) return qfail(q, flagcxInvalidArgument, "%s: count overflows", who);
  const uint64_t bytes = count * ts;
  memset(&e, 0, sizeof(e));
  const uintptr_t mis = (uintptr_t)dst & 15u;
  e.flags = kQueueFlagAligned;
  for (int j = 0; j < k; j++) {
    const uintptr_t s = (uintptr_t)srcs[j];
    if (!s) return qfail(q, flagcxInvalidArgument, "%s: sendbuffs[%d] is NULL", who, j);
    if (s % ts) return qfail(q, flagcxInvalidArgument, "%s: sendbuffs[%d] not aligned to its element size", who, j);
    if (s != (uintptr_t)dst && overlaps(s, (uintptr_t)dst, bytes, bytes))
      return qfail(q, flagcxInvalidArgument, "%s: recvbuff partially overlaps sendbuffs[%d]", who, j);
    if ((s & 15u) != mis) e.flags &= ~(uint32_t)kQueueFlagAligned;
    e.src[j] = (uint64_t)s;
  }
  e.dst = (uint64_t)(uintptr_t)dst;
  const uint64_t perVec = 16 / ts;
  uint64_t head = ((16u - mis) & 15u) / ts;
  if (head > count) head = count;
  e.head = (uint32_t)head;
  e.nvec = (count - head) / perVec;
  e.tail = (uint32_t)(count - head - e.nvec * perVec);
  e.k = (uint32_t)k;
  *empty = false;
  return flagcxSuccess;
}

// Waits until no consumer kernel is on the GPU.
flagcxResult_t joinConsumer(flagcxLocalReduceFifo *q) {
  const hipError_t e = hipStreamSynchronize(q->stream);
  return e == hipSuccess ? flagcxSuccess
                         : qfail(q, flagcxUnhandledDeviceError, "flagcxLocalReduceFifo: %s", hipGetErrorString(e));
}

} // namespace

#pragma GCC visibility push(default)
extern "C" {

flagcxResult_t flagcxLocalReduceFifoCreate(flagcxLocalReduceFifo_t *fifo, int capacity, int maxRanks,
                                           flagcxDataType_t datatype, flagcxRedOp_t op) {
  if (!fifo) return flagcxInvalidArgument;
  *fifo = nullptr;
  int dt, rop;
  memcpy(&dt, &datatype, sizeof(int));
  memcpy(&rop, &op, sizeof(int));
  const size_t ts = flagcxLocalGetDataTypeSize((flagcxDataType_t)(dt >= 0 && dt < (int)flagcxNumTypes ? dt : 0));
  if (dt < 0 || dt >= (int)flagcxNumTypes || !ts || !reduceQueueLauncherFor(dt)) return flagcxInvalidArgument;
  if (rop < 0 || rop >= (int)flagcxNumRedOps) return flagcxInvalidArgument;
  if (capacity < 1 || capacity > 65536 || maxRanks < 1 || maxRanks > 8) return flagcxInvalidArgument;
  flagcxLocalReduceFifo *q = new (std::nothrow) flagcxLocalReduceFifo;
  if (!q) return flagcxSystemError;
  q->capacity = (uint32_t)capacity;
  q->maxRanks = maxRanks;
  q->dtype = dt;
  q->op = rop;
  q->typeSize = ts;
  // Measured on MI355X (128 x 4 MiB chunks per input, units drawn by ticket): with the
  // workers' units of 8 / 4 / 1 KiB per input for up to 2 / up to 4 / more inputs, about
  // 64-100 KiB of loads in flight per CU are enough (two inputs 6.05 / 6.0 / 5.8 / 5.6 TB/s at
  // 8 / 10 / 12 / 14 wavefronts per CU, three 5.9 / 6.05 / 6.0 / 5.7, four 6.35 / 6.0 / 5.8 / 5.6,
  // six 4.7 / 5.4 / 5.8 / 6.0, eight 5.5 / 5.9 / 6.1 / 6.1); never more than half a CU's
  // slots, so that residency does not depend on the last slot being free.  (A limit on
  // the inputs a worker has in flight, which the launched kernels use for large
  // reduces, only costs here.)
  static const int kWaves[9] = {8, 8, 8, 10, 8, 14, 14, 12, 12};
  q->wavesPerCU = kWaves[maxRanks];
  const DeviceInfo &info = deviceInfo();
  q->maxGrid = (unsigned)info.numCU * 16u;
  const size_t hostBytes = kQueueHeaderWords * sizeof(uint64_t) + (size_t)capacity * sizeof(QueueEntry);
  const size_t devBytes = (size_t)capacity * sizeof(QueueEntry) + 128 + (size_t)q->maxGrid * sizeof(uint64_t) +
                          (size_t)kQueueMaxTicketCounters * kQueueTicketStride * sizeof(uint64_t);
  void *host = nullptr;
  hipError_t e = hipHostMalloc(&host, hostBytes, hipHostMallocMapped);
  if (e == hipSuccess) e = hipMalloc(&q->devBlock, devBytes);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&q->stream, hipStreamNonBlocking);
  if (e != hipSuccess) {
    if (host) (void)hipHostFree(host);
    if (q->devBlock) (void)hipFree(q->devBlock);
    delete q;
    return flagcxUnhandledDeviceError;
  }
  memset(host, 0, hostBytes);
  q->header = static_cast<uint64_t *>(host);
  q->header[kQueueCapacity] = (uint64_t)capacity;
  q->hostEntries = reinterpret_cast<QueueEntry *>(q->header + kQueueHeaderWords);
  q->devEntries = static_cast<QueueEntry *>(q->devBlock);
  q->devProduced = reinterpret_cast<uint64_t *>(q->devEntries + capacity);
  q->progress = reinterpret_cast<uint32_t *>(q->devProduced + 16);
  q->tickets = q->devProduced + 16 + q->maxGrid;
  *fifo = q;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoStart(flagcxLocalReduceFifo_t q) {
  if (!q) return flagcxInvalidArgument;
  std::lock_guard<std::mutex> lock(q->mu);
  const char *who = "flagcxLocalReduceFifoStart";
  if (q->started) {
    if (alive(headerLoad(q, kQueueState))) return qfail(q, flagcxInvalidUsage, "%s: already running", who);
    q->started = false; // the previous consumer timed out
  }
  flagcxResult_t r = joinConsumer(q);
  if (r != flagcxSuccess) return r;
  q->produced = 0;
  q->lastAfterAll = 0;
  q->header[kQueueConsumed] = 0;
  __atomic_store_n(q->header + kQueueProduced, (uint64_t)0, __ATOMIC_RELEASE);
  r = launchConsumer(q, 0, who);
  if (r != flagcxSuccess) return r;
  q->started = true;
  q->stopSent = false;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoEnqueueReduce(flagcxLocalReduceFifo_t q, const void *const *sendbuffs, int nranks,
                                                  void *recvbuff, size_t count, uint64_t *ticket) {
  if (!q) return flagcxInvalidArgument;
  const char *who = "flagcxLocalReduceFifoEnqueueReduce";
  if (!sendbuffs) return qfail(q, flagcxInvalidArgument, "%s: sendbuffs is NULL", who);
  std::lock_guard<std::mutex> lock(q->mu);
  QueueEntry e;
  bool empty;
  flagcxResult_t r = buildEntry(q, sendbuffs, nranks, recvbuff, count, e, &empty, who);
  if (r != flagcxSuccess) return r;
  if (empty) {
    if (ticket) *ticket = q->produced;
    return flagcxSuccess;
  }
  return appendEntry(q, e, ticket, who);
}

flagcxResult_t flagcxLocalReduceFifoEnqueue(flagcxLocalReduceFifo_t q, const flagcxLocalReduceTrigger *trigger,
                                            uint64_t *ticket) {
  if (!q) return flagcxInvalidArgument;
  const char *who = "flagcxLocalReduceFifoEnqueue";
  if (!trigger) return qfail(q, flagcxInvalidArgument, "%s: trigger is NULL", who);
  const uint64_t *v = trigger->value;
  const int dt = (int)((v[3] >> 48) & 0xf), op = (int)((v[3] >> 52) & 0xf);
  if (dt != q->dtype || op != q->op)
    return qfail(q, flagcxInvalidArgument, "%s: trigger datatype %d / redop %d differ from the queue's", who, dt, op);
  // addr3 = OP(addr1, addr2): fold order acc = addr2; acc = OP(addr1, acc)
  const void *srcs[2] = {(const void *)(uintptr_t)v[1], (const void *)(uintptr_t)v[0]};
  std::lock_guard<std::mutex> lock(q->mu);
  if (q->maxRanks < 2) return qfail(q, flagcxInvalidArgument, "%s: the queue was created for one input", who);
  QueueEntry e;
  bool empty;
  flagcxResult_t r = buildEntry(q, srcs, 2, (void *)(uintptr_t)v[2], v[3] & 0xffffffffull, e, &empty, who);
  if (r != flagcxSuccess) return r;
  if (empty) {
    if (ticket) *ticket = q->produced;
    return flagcxSuccess;
  }
  return appendEntry(q, e, ticket, who);
}

flagcxResult_t flagcxLocalReduceFifoQuery(flagcxLocalReduceFifo_t q, uint64_t *produced, uint64_t *consumed,
                                          int *state) {
  if (!q) return flagcxInvalidArgument;
  if (consumed) *consumed = headerLoad(q, kQueueConsumed);
  if (produced) *produced = producedLoad(q);
  if (state) *state = (int)headerLoad(q, kQueueState);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoWait(flagcxLocalReduceFifo_t q, uint64_t ticket) {
  if (!q) return flagcxInvalidArgument;
  const char *who = "flagcxLocalReduceFifoWait";
  if (ticket > producedLoad(q))
    return qfail(q, flagcxInvalidArgument, "%s: ticket %lld has not been handed out", who, (long long)ticket);
  for (;;) {
    if (headerLoad(q, kQueueConsumed) >= ticket) return flagcxSuccess;
    const uint64_t state = headerLoad(q, kQueueState);
    if (!alive(state)) {
      if (headerLoad(q, kQueueConsumed) >= ticket) return flagcxSuccess;
      return qfail(q, state == kQueueTimedOut ? flagcxInternalError : flagcxInvalidUsage,
                   "%s: the consumer is not running (state %lld) and entry %lld was not reached", who,
                   (long long)state, (long long)ticket);
    }
    sched_yield();
  }
}

flagcxResult_t flagcxLocalReduceFifoStop(flagcxLocalReduceFifo_t q) {
  if (!q) return flagcxInvalidArgument;
  std::lock_guard<std::mutex> lock(q->mu);
  if (!q->started) return flagcxSuccess;
  const char *who = "flagcxLocalReduceFifoStop";
  if (!q->stopSent && alive(headerLoad(q, kQueueState))) {
    QueueEntry e;
    memset(&e, 0, sizeof(e)); // k = 0
    // a full ring drains by itself: entries ahead of the stop entry finish first
    for (;;) {
      if (!alive(headerLoad(q, kQueueState))) break;
      if (q->produced - headerLoad(q, kQueueConsumed) < q->capacity) {
        memcpy(q->hostEntries + q->produced % q->capacity, &e, sizeof(e));
        bool wasParked;
        (void)publishEntry(q, who, &wasParked);
        q->stopSent = true;
        if (wasParked) {
          // no consumer is left to read the stop entry, and nothing was outstanding
          __atomic_store_n(q->header + kQueueConsumed, q->produced, __ATOMIC_RELEASE);
          flagcxResult_t r = joinConsumer(q); // the parked kernel's last stores are done
          if (r != flagcxSuccess) return r;
          __atomic_store_n(q->header + kQueueState, (uint64_t)kQueueStopped, __ATOMIC_RELEASE);
        }
        break;
      }
      sched_yield();
    }
  }
  const uint64_t want = q->produced;
  flagcxResult_t r = joinConsumer(q);
  q->started = false;
  q->stopSent = false;
  if (r != flagcxSuccess) return r;
  const uint64_t state = headerLoad(q, kQueueState);
  if (state == kQueueTimedOut || headerLoad(q, kQueueConsumed) < want)
    return qfail(q, flagcxInternalError,
                 "%s: the consumer gave up after its spin limit with %lld of %lld entries done", who,
                 (long long)headerLoad(q, kQueueConsumed), (long long)want);
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoDestroy(flagcxLocalReduceFifo_t q) {
  if (!q) return flagcxSuccess;
  flagcxResult_t r = flagcxLocalReduceFifoStop(q);
  hipError_t e = hipStreamDestroy(q->stream);
  hipError_t e2 = hipFree(q->devBlock);
  hipError_t e3 = hipHostFree(q->header);
  delete q;
  if (e != hipSuccess || e2 != hipSuccess || e3 != hipSuccess) return flagcxUnhandledDeviceError;
  return r;
}

flagcxResult_t flagcxLocalReduceFifoSetWaves(flagcxLocalReduceFifo_t q, int wavesPerCU) {
  if (!q) return flagcxInvalidArgument;
  std::lock_guard<std::mutex> lock(q->mu);
  if (wavesPerCU < 1 || wavesPerCU > 16)
    return qfail(q, flagcxInvalidArgument, "flagcxLocalReduceFifoSetWaves: %d outside [1, 16]", wavesPerCU);
  if (q->started) return qfail(q, flagcxInvalidUsage, "flagcxLocalReduceFifoSetWaves: the queue is started");
  q->wavesPerCU = wavesPerCU;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoSetLinger(flagcxLocalReduceFifo_t q, int64_t polls) {
  if (!q) return flagcxInvalidArgument;
  std::lock_guard<std::mutex> lock(q->mu);
  if (polls < 0) return qfail(q, flagcxInvalidArgument, "flagcxLocalReduceFifoSetLinger: negative");
  if (q->started) return qfail(q, flagcxInvalidUsage, "flagcxLocalReduceFifoSetLinger: the queue is started");
  q->linger = polls;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoSetOwnQueue(flagcxLocalReduceFifo_t q, int own) {
  const char *who = "flagcxLocalReduceFifoSetOwnQueue";
  if (!q) return flagcxInvalidArgument;
  std::lock_guard<std::mutex> lock(q->mu);
  if (q->started) return qfail(q, flagcxInvalidUsage, "%s: the queue is started", who);
  // A stream with a CU mask does not come from the runtime's pool of hardware queues (the
  // mask is a property of the queue): with every CU in the mask it differs from an ordinary
  // stream only in that no other stream is ever mapped to its hardware queue, and in that
  // the runtime creates such streams blocking.
  hipStream_t fresh = nullptr;
  hipError_t e;
  if (own) {
    uint32_t mask[32];
    for (int i = 0; i < 32; i++) mask[i] = 0xffffffffu;
    int words = (deviceInfo().numCU + 31) / 32;
    if (words < 1) words = 1;
    if (words > 32) words = 32;
    e = hipExtStreamCreateWithCUMask(&fresh, (uint32_t)words, mask);
  } else {
    e = hipStreamCreateWithFlags(&fresh, hipStreamNonBlocking);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return qfail(q, flagcxUnhandledDeviceError, "%s: %s", who, hipGetErrorString(e));
  }
  (void)hipStreamSynchronize(q->stream);
  (void)hipStreamDestroy(q->stream);
  q->stream = fresh;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoSetWindow(flagcxLocalReduceFifo_t q, size_t bytes) {
  if (!q) return flagcxInvalidArgument;
  std::lock_guard<std::mutex> lock(q->mu);
  if (bytes == 0) return qfail(q, flagcxInvalidArgument, "flagcxLocalReduceFifoSetWindow: zero");
  if (q->started) return qfail(q, flagcxInvalidUsage, "flagcxLocalReduceFifoSetWindow: the queue is started");
  q->windowBytes = bytes;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalReduceFifoGetType(flagcxLocalReduceFifo_t q, flagcxDataType_t *datatype, flagcxRedOp_t *op,
                                            int *maxRanks) {
  if (!q) return flagcxInvalidArgument;
  if (datatype) *datatype = (flagcxDataType_t)q->dtype;
  if (op) *op = (flagcxRedOp_t)q->op;
  if (maxRanks) *maxRanks = q->maxRanks;
  return flagcxSuccess;
}

const char *flagcxLocalReduceFifoGetLastError(flagcxLocalReduceFifo_t q) { return q ? q->lastError : ""; }

flagcxResult_t flagcxLocalReduceFifoGetGrid(flagcxLocalReduceFifo_t q, unsigned *workgroups) {
  if (!q || !workgroups) return flagcxInvalidArgument;
  *workgroups = q->grid;
  return flagcxSuccess;
}

} // extern "C"
#pragma GCC visibility pop
