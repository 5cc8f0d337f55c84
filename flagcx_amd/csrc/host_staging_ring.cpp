// host_staging_ring.cpp - the staging pipeline either side of the local reduce.
//
// The reference moves every message between ranks through a ring of
// FLAGCX_P2P_STEPS (16) slots of FLAGCX_P2P_CHUNKSIZE (4 MiB)
// (flagcx/core/p2p.h:11-15, same numbers in flagcx/core/net.h:19-22): the sender's
// proxy copies min(chunk, size - copied) bytes into slot (step & 15) and bumps
// sendHead once the copy's event has fired (flagcx/core/p2p.cc:75-107); the
// receiver copies the slot out and bumps recvTail, which frees the slot for step
// + 16 (p2p.cc:170-205).  Here both sides live on one GPU: a producer stream
// plays the sender's proxy, a consumer stream the receiver's, and the head / tail
// counters become one "filled" and one "freed" HIP event per slot.  The consumer
// either copies the slot out (send/recv) or - the reduce-scatter form - folds the
// slots of all peers and the local slice straight into the output, so the reduce
// of chunk i overlaps the staging copies of chunk i+1.
//
// Ring memory belongs to the caller (steps * npeers * chunkBytes); creating the
// object allocates only the events.
#include "../../include/flagcx_amd.h"

#include <hip/hip_runtime.h>
#include <sched.h>

#include <vector>

struct flagcxLocalRing {
  char *buffer = nullptr;
  size_t chunkBytes = 0;
  int steps = 0, npeers = 0;
  std::vector<hipEvent_t> filled, freed;
  hipEvent_t start = nullptr;
};

namespace {

inline hipStream_t hipOf(flagcxStream_t s) { return s ? *reinterpret_cast<hipStream_t *>(s) : nullptr; }

#define RCHECK(call)                                                           \
  do {                                                                         \
    flagcxResult_t r_ = (call);                                                \
    if (r_ != flagcxSuccess) return r_;                                        \
  } while (0)
#define HCHECK(call)                                                           \
  do {                                                                         \
    if ((call) != hipSuccess) return flagcxUnhandledDeviceError;               \
  } while (0)

inline char *slotOf(flagcxLocalRing *r, size_t step, int peer) {
  return r->buffer + ((step % (size_t)r->steps) * (size_t)r->npeers + (size_t)peer) * r->chunkBytes;
}

// Steps handed over together.  A hand-over between the producer and the consumer
// costs about as much as moving a 4 MiB step (an event crossing streams, or a
// polled one), so full steps travel in groups of up to eight: half the ring, which
// leaves two groups in flight, where the slots of a group are one contiguous region
// (every peer region in use).  The last, ragged step always travels alone.
constexpr size_t kGroup = 8;
inline size_t groupAt(const flagcxLocalRing *r, int regions, size_t step, size_t nsteps, size_t size) {
  if (regions != r->npeers) return 1;
  size_t g = kGroup;
  while (g > 1 && ((size_t)r->steps % g || (size_t)r->steps < 2 * g)) g >>= 1;
  if (g == 1 || step % g) return 1;
  size_t m = nsteps - step < g ? nsteps - step : g;
  // only whole chunks: a ragged last step leaves the group
  if ((step + m) * r->chunkBytes > size) m--;
  // one pack launch takes 64 source regions
  while (m > 1 && m * (size_t)regions > 64) m--;
  return m ? m : 1;
}

} // namespace

#pragma GCC visibility push(default)
extern "C" {

flagcxResult_t flagcxLocalRingCreate(flagcxLocalRing **ring, void *ringBuffer, size_t ringBytes, int npeers,
                                     size_t chunkBytes, int steps) {
  if (!ring || !ringBuffer || npeers < 1 || npeers >= FLAGCX_LOCAL_MAX_RANKS) return flagcxInvalidArgument;
  if (chunkBytes == 0) chunkBytes = FLAGCX_LOCAL_CHUNKSIZE;
  if (steps == 0) steps = FLAGCX_LOCAL_STEPS;
  if (steps < 1 || steps > 1024 || (chunkBytes & 15u)) return flagcxInvalidArgument;
  if (ringBytes < (size_t)steps * (size_t)npeers * chunkBytes) return flagcxInvalidArgument;
  flagcxLocalRing *r = nullptr;
  try { // nothing may leave an extern "C" function by exception
    r = new flagcxLocalRing();
    r->filled.resize(steps);
    r->freed.resize(steps);
  } catch (...) {
    delete r;
    return flagcxSystemError;
  }
  r->buffer = static_cast<char *>(ringBuffer);
  r->chunkBytes = chunkBytes;
  r->steps = steps;
  r->npeers = npeers;
  bool ok = hipEventCreateWithFlags(&r->start, hipEventDisableTiming) == hipSuccess;
  for (int i = 0; ok && i < steps; i++) {
    ok = hipEventCreateWithFlags(&r->filled[i], hipEventDisableTiming) == hipSuccess &&
         hipEventCreateWithFlags(&r->freed[i], hipEventDisableTiming) == hipSuccess;
  }
  if (!ok) {
    delete r; // events created so far are few; the process is in trouble anyway
    return flagcxUnhandledDeviceError;
  }
  *ring = r;
  return flagcxSuccess;
}

flagcxResult_t flagcxLocalRingDestroy(flagcxLocalRing *r) {
  if (!r) return flagcxSuccess;
  for (auto e : r->filled) if (e) (void)hipEventDestroy(e);
  for (auto e : r->freed) if (e) (void)hipEventDestroy(e);
  if (r->start) (void)hipEventDestroy(r->start);
  delete r;
  return flagcxSuccess;
}

// One message through the ring: producer copies src -> slot, consumer slot -> dst.
flagcxResult_t flagcxLocalRingSendRecv(flagcxLocalRing *r, void *dst, const void *src, size_t size,
                                       flagcxStream_t copyStream, flagcxStream_t stream) {
  if (!r || !copyStream || !stream) return flagcxInvalidArgument;
  if (size == 0) return flagcxSuccess;
  if (!dst || !src) return flagcxInvalidArgument;
  hipStream_t ps = hipOf(copyStream), cs = hipOf(stream);
  HCHECK(hipEventRecord(r->start, cs)); // what the consumer stream produced so far is the sender's input
  HCHECK(hipStreamWaitEvent(ps, r->start, 0));
  const size_t nsteps = (size + r->chunkBytes - 1) / r->chunkBytes; // chunkSteps (flagcx/core/group.cc:179-181)
  for (size_t step = 0; step < nsteps;) {
    const size_t m = groupAt(r, 1, step, nsteps, size); // whole steps in consecutive slots share one hand-over
    const int slot = (int)(step % (size_t)r->steps);
    const size_t off = step * r->chunkBytes;
    const size_t n = m > 1 ? m * r->chunkBytes : (size - off < r->chunkBytes ? size - off : r->chunkBytes);
    if (step >= (size_t)r->steps) HCHECK(hipStreamWaitEvent(ps, r->freed[slot], 0)); // recvTail > copied
    RCHECK(flagcxLocalMemcpy(slotOf(r, step, 0), (const char *)src + off, n, copyStream));
    HCHECK(hipEventRecord(r->filled[slot], ps));                                       // sendHead
    HCHECK(hipStreamWaitEvent(cs, r->filled[slot], 0));
    RCHECK(flagcxLocalMemcpy((char *)dst + off, slotOf(r, step, 0), n, stream));
    HCHECK(hipEventRecord(r->freed[slot], cs));                                        // recvTail
    step += m;
  }
  return flagcxSuccess;
}

// Rank `rank`'s reduce-scatter shard with the nranks-1 peers' slices arriving
// through the ring, chunk by chunk; result identical to flagcxLocalReduceScatter.
flagcxResult_t flagcxLocalRingReduceScatter(flagcxLocalRing *r, const void *const *sendbuffs, int nranks,
                                            int rank, void *recvbuff, size_t recvcount,
                                            flagcxDataType_t datatype, flagcxRedOp_t op,
                                            flagcxStream_t copyStream, flagcxStream_t stream) {
  if (!r || !sendbuffs || !copyStream || !stream) return flagcxInvalidArgument;
  if (nranks < 1 || nranks > FLAGCX_LOCAL_MAX_RANKS || rank < 0 || rank >= nranks) return flagcxInvalidArgument;
  if (nranks - 1 > r->npeers) return flagcxInvalidArgument;
  const size_t ts = flagcxLocalGetDataTypeSize(datatype);
  if (!ts || (r->chunkBytes % ts)) return flagcxInvalidArgument;
  if (recvcount == 0) return flagcxSuccess;
  if (nranks == 1) // nothing to stage (flagcx/service/bootstrap.cc:856-861)
    return flagcxLocalReduceScatter(sendbuffs, 1, 0, recvbuff, recvcount, datatype, op, stream);
  hipStream_t ps = hipOf(copyStream), cs = hipOf(stream);
  HCHECK(hipEventRecord(r->start, cs));
  HCHECK(hipStreamWaitEvent(ps, r->start, 0));
  const size_t size = recvcount * ts;
  const size_t nsteps = (size + r->chunkBytes - 1) / r->chunkBytes;
  const void *peerSrc[kGroup * FLAGCX_LOCAL_MAX_RANKS];
  const void *ordered[kGroup][FLAGCX_LOCAL_MAX_RANKS];
  flagcxLocalReduceDesc descs[kGroup];
  for (size_t step = 0; step < nsteps;) {
    const size_t m = groupAt(r, nranks - 1, step, nsteps, size); // steps step .. step+m-1 share one hand-over
    const int slot = (int)(step % (size_t)r->steps);
    const size_t off = step * r->chunkBytes;
    const size_t n = m > 1 || size - off >= r->chunkBytes ? r->chunkBytes : size - off;
    // ring order rank+1, ..., rank: the first nranks-1 are peers, the last is local
    for (size_t i = 0; i < m; i++) {
      for (int j = 0; j < nranks - 1; j++) {
        const int peer = (rank + 1 + j) % nranks;
        peerSrc[i * (size_t)(nranks - 1) + j] = (const char *)sendbuffs[peer] + (size_t)rank * size + off + i * n;
        ordered[i][j] = slotOf(r, step + i, j);
      }
      ordered[i][nranks - 1] = (const char *)sendbuffs[rank] + (size_t)rank * size + off + i * n;
    }
    if (step >= (size_t)r->steps) HCHECK(hipStreamWaitEvent(ps, r->freed[slot], 0));
    // the peer regions of a slot, and the slots of a group, are contiguous: one launch stages them all
    RCHECK(flagcxLocalPackList(slotOf(r, step, 0), peerSrc, (int)(m * (size_t)(nranks - 1)), n, copyStream));
    if (n != r->chunkBytes) // ragged last chunk: regions are n apart after a pack
      for (int j = 0; j < nranks - 1; j++) ordered[0][j] = slotOf(r, step, 0) + (size_t)j * n;
    HCHECK(hipEventRecord(r->filled[slot], ps));
    HCHECK(hipStreamWaitEvent(cs, r->filled[slot], 0));
    for (size_t i = 0; i < m; i++) {
      descs[i].sendbuffs = ordered[i];
      descs[i].recvbuff = (char *)recvbuff + off + i * n;
      descs[i].count = n / ts;
    }
    if (m == 1)
      RCHECK(flagcxLocalReduce(ordered[0], nranks, (char *)recvbuff + off, n / ts, datatype, op, stream));
    else
      RCHECK(flagcxLocalReduceBatch(descs, (int)m, nranks, datatype, op, stream));
    HCHECK(hipEventRecord(r->freed[slot], cs));
    step += m;
  }
  return flagcxSuccess;
}

// The same shard with the host in the role of the reference's proxy thread, which
// never makes one stream wait for another: it issues a step's copy, records an
// event, polls it with eventQuery and only then hands the step on
// (flagcx/core/p2p.cc:75-107,170-205).  Here "hands on" is an entry in the resident
// reduce queue, and a slot is free again when that entry's ticket is consumed.
// Blocks until the shard is complete.
flagcxResult_t flagcxLocalRingReduceScatterFifo(flagcxLocalRing *r, flagcxLocalReduceFifo_t fifo,
                                                const void *const *sendbuffs, int nranks, int rank,
                                                void *recvbuff, size_t recvcount, flagcxStream_t copyStream) {
  if (!r || !fifo || !sendbuffs || !copyStream) return flagcxInvalidArgument;
  if (nranks < 1 || nranks > FLAGCX_LOCAL_MAX_RANKS || rank < 0 || rank >= nranks) return flagcxInvalidArgument;
  if (nranks - 1 > r->npeers) return flagcxInvalidArgument;
  flagcxDataType_t datatype;
  flagcxRedOp_t op;
  int maxRanks = 0;
  RCHECK(flagcxLocalReduceFifoGetType(fifo, &datatype, &op, &maxRanks));
  if (nranks > maxRanks) return flagcxInvalidArgument;
  const size_t ts = flagcxLocalGetDataTypeSize(datatype);
  if (!ts || (r->chunkBytes % ts)) return flagcxInvalidArgument;
  if (recvcount == 0) return flagcxSuccess;
  hipStream_t ps = hipOf(copyStream);
  const size_t size = recvcount * ts;
  const size_t nsteps = (size + r->chunkBytes - 1) / r->chunkBytes;
  const size_t depth = (size_t)r->steps;
  uint64_t ticket[1024] = {0}; // per slot (a ring has at most 1024): ticket of the entry that reads it
  int lead[1024] = {0};        // per slot: the slot whose `filled` event covers its copy
  const void *peerSrc[kGroup * FLAGCX_LOCAL_MAX_RANKS];
  const void *ordered[FLAGCX_LOCAL_MAX_RANKS];
  size_t copied = 0, handed = 0; // steps whose copy is issued / whose reduce is enqueued
  uint64_t lastTicket = 0, consumed = 0;
  while (handed < nsteps) {
    const size_t copiedBefore = copied, handedBefore = handed;
    int state = 0;
    RCHECK(flagcxLocalReduceFifoQuery(fifo, nullptr, &consumed, &state));
    // a consumer that has left for good (stopped, or timed out on its spin bound)
    // frees no more slots: give up instead of waiting for `consumed` to move
    if (state != FLAGCX_LOCAL_REDUCE_FIFO_RUNNING && state != FLAGCX_LOCAL_REDUCE_FIFO_PARKED && handed > 0 &&
        consumed < lastTicket)
      return flagcxInternalError;
    // issue copies into free slots (sendHead side), a group of steps per launch and event
    while (copied < nsteps) {
      const size_t m = groupAt(r, nranks - 1, copied, nsteps, size);
      const size_t last = copied + m - 1; // tickets grow with the step: the last slot of the group frees last
      if (!(last < depth || (last - depth < handed && consumed >= ticket[last % depth]))) break;
      const size_t off = copied * r->chunkBytes;
      const size_t n = m > 1 || size - off >= r->chunkBytes ? r->chunkBytes : size - off;
      for (size_t i = 0; i < m; i++)
        for (int j = 0; j < nranks - 1; j++)
          peerSrc[i * (size_t)(nranks - 1) + j] =
              (const char *)sendbuffs[(rank + 1 + j) % nranks] + (size_t)rank * size + off + i * n;
      if (nranks > 1)
        RCHECK(flagcxLocalPackList(slotOf(r, copied, 0), peerSrc, (int)(m * (size_t)(nranks - 1)), n, copyStream));
      HCHECK(hipEventRecord(r->filled[copied % depth], ps));
      for (size_t i = 0; i < m; i++) lead[(copied + i) % depth] = (int)(copied % depth);
      copied += m;
    }
    // hand on, in order, every step whose copy has completed (recvTail side)
    while (handed < copied) {
      const hipError_t q = hipEventQuery(r->filled[lead[handed % depth]]);
      if (q == hipErrorNotReady) break;
      if (q != hipSuccess) return flagcxUnhandledDeviceError;
      const size_t off = handed * r->chunkBytes;
      const size_t n = size - off < r->chunkBytes ? size - off : r->chunkBytes;
      for (int j = 0; j < nranks - 1; j++) ordered[j] = slotOf(r, handed, 0) + (size_t)j * n;
      ordered[nranks - 1] = (const char *)sendbuffs[rank] + (size_t)rank * size + off;
      const flagcxResult_t e =
          flagcxLocalReduceFifoEnqueueReduce(fifo, ordered, nranks, (char *)recvbuff + off, n / ts, &lastTicket);
      if (e == flagcxInProgress) break; // queue full: its entries drain by themselves
      if (e != flagcxSuccess) return e;
      ticket[handed % depth] = lastTicket;
      handed++;
    }
    if (copied == copiedBefore && handed == handedBefore) sched_yield(); // nothing moved: let the copies and the consumer run
  }
  return flagcxLocalReduceFifoWait(fifo, lastTicket);
}

} // extern "C"
#pragma GCC visibility pop
