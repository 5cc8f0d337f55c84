/*
 * flagcx_amd.h - C ABI of the MI355X (gfx950) local reduce / chunk copy library.
 *
 * Every entry point is `extern "C"`, takes plain pointers and sizes, allocates
 * nothing, never calls hipSetDevice, and enqueues its work asynchronously on the
 * caller's stream.  Return values are flagcxResult_t numbers.
 *
 * Conventions shared by all entry points
 *   - "sendbuffs" is a HOST array of `nranks` DEVICE pointers: buffer j holds what
 *     simulated rank j contributes.  The array is read during the call only.
 *   - stream is the reference's opaque handle (flagcx/include/flagcx.h:112); on AMD
 *     it points at a struct whose first member is the hipStream_t
 *     (flagcx/adaptor/include/amd_adaptor.h:14-16).  NULL selects the legacy default
 *     stream and the call blocks until the work has finished, like the reference's
 *     hipAdaptorDeviceMemcpy / Memset (flagcx/adaptor/device/hip_adaptor.cc:16-41).
 *   - recvbuff may be the same address as one sendbuff (element i is read before
 *     element i is written); any other overlap is flagcxInvalidArgument.
 *   - buffers need only be aligned to the element size (byte aligned for copies).
 *   - count == 0 / size == 0 is flagcxSuccess and launches nothing.
 */
#ifndef FLAGCX_AMD_H_
#define FLAGCX_AMD_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------------- */
/* Enums: numeric values are ABI and equal flagcx/include/flagcx.h:12-57,78-88 */
/* If the reference's own flagcx.h was included first, its definitions are    */
/* used and these are skipped.                                                */
/* ------------------------------------------------------------------------- */
#ifndef FLAGCX_H_

typedef enum {
  flagcxSuccess = 0,
  flagcxUnhandledDeviceError = 1,
  flagcxSystemError = 2,
  flagcxInternalError = 3,
  flagcxInvalidArgument = 4,
  flagcxInvalidUsage = 5,
  flagcxRemoteError = 6,
  flagcxInProgress = 7,
  flagcxUnhandledCCLError = 8,
  flagcxNotSupported = 9,
  flagcxNumResults = 10
} flagcxResult_t;

typedef enum {
  flagcxInt8 = 0, flagcxChar = 0,
  flagcxUint8 = 1,
  flagcxInt32 = 2, flagcxInt = 2,
  flagcxUint32 = 3,
  flagcxInt64 = 4,
  flagcxUint64 = 5,
  flagcxFloat16 = 6, flagcxHalf = 6,
  flagcxFloat32 = 7, flagcxFloat = 7,
  flagcxFloat64 = 8, flagcxDouble = 8,
  flagcxBfloat16 = 9,
  flagcxNumTypes = 10
} flagcxDataType_t;

typedef enum {
  flagcxSum = 0,
  flagcxProd = 1,
  flagcxMax = 2,
  flagcxMin = 3,
  flagcxAvg = 4,
  flagcxRedNoOp = 5,
  flagcxNumRedOps = 5
} flagcxRedOp_t;

typedef enum {
  flagcxCommOpSend = 0,
  flagcxCommOpRecv = 1,
  flagcxCommOpBroadcast = 2,
  flagcxCommOpGather = 3,
  flagcxCommOpScatter = 4,
  flagcxCommOpReduce = 5,
  flagcxCommOpAllReduce = 6,
  flagcxCommOpAllGather = 7,
  flagcxCommOpReduceScatter = 8,
  flagcxCommOpAlltoAll = 9,
  flagcxCommOpAlltoAllv = 10,
  flagcxCommNoOp = 11,
  flagcxNumCommOps = 12
} flagcxCommOp_t;

typedef enum {
  flagcxMemcpyHostToDevice = 0,
  flagcxMemcpyDeviceToHost = 1,
  flagcxMemcpyDeviceToDevice = 2
} flagcxMemcpyType_t;

/* Opaque in the reference (flagcx.h:112); layout fixed by amd_adaptor.h:14-16. */
typedef struct flagcxStream *flagcxStream_t;

#endif /* FLAGCX_H_ */

/* Bytes per element, 0 for an unknown enum value: the table of
 * getFlagcxDataTypeSize (flagcx/flagcx.cc:30-61) under a name that does not clash
 * with the reference's own export when both libraries are loaded. */
size_t flagcxLocalGetDataTypeSize(flagcxDataType_t dtype);

/* Largest number of simulated ranks (input buffers) one call accepts. */
#define FLAGCX_LOCAL_MAX_RANKS 64

/* Pipeline constants of the reference's staging rings:
 * flagcx/core/p2p.h:11-15 and flagcx/core/net.h:19-22. */
#define FLAGCX_LOCAL_CHUNKSIZE (4ULL * 1024 * 1024)
#define FLAGCX_LOCAL_STEPS 16

/* ------------------------------------------------------------------------- */
/* Library                                                                    */
/* ------------------------------------------------------------------------- */

/* Caches the properties of the current device (CU count) and looks up where the
 * library's static staging area lives on it (flagcxLocalStagedReduceScatterNoAlloc).
 * Optional: every entry point does its part on first use.  Call it once per device,
 * with that device current, before capturing graphs there.  Thread-safe. */
flagcxResult_t flagcxLocalInit(void);

/* Static string for a result code (never NULL). */
const char *flagcxLocalGetErrorString(flagcxResult_t result);

/* Text of the last failure seen by the calling thread ("" if none). */
const char *flagcxLocalGetLastError(void);

/* Where to put `nbuffers` buffers of `bytes` each inside one allocation so that
 * equal offsets into them fall into different HBM channel groups (MI355X has 32,
 * chosen by address bits 10..14, 18..22 and 25..29): KiB-aligned addresses inside
 * [pool, pool + poolbytes), in increasing order, at most 64 KiB of padding each
 * (beyond 32 buffers every run of 32 shares the groups out again).
 * The callers that allocate the ranks' staging / scratch buffers
 * (flagcx/core/c2c_algo.cc:2121-2137) can place them this way: an 8-input reduce
 * of 256 MiB per input runs at 87 % of the HBM peak over buffers placed by this
 * call and at 85-86 % over buffers that all start in the same group (e.g. 258 MiB
 * apart, where a caching allocator puts 256 MiB buffers).  Host-only, no device
 * access. */
flagcxResult_t flagcxLocalPlaceBuffers(void *pool, size_t poolbytes, size_t bytes, int nbuffers, void **buffers);

/* Launch-shape knobs, in the spirit of the reference's FLAGCX_* tuning variables.
 * Tune: how many one-wavefront workgroups may share a CU for a reduce of `nranks`
 * inputs (1..8; 0 selects the copy kernels).  wavesPerCU == 0 removes the cap,
 * -1 (the default, and what GetTune then reports) lets every launch choose from
 * the values measured on MI355X.
 * TuneLoads: of how many of its `nranks` inputs (2..8) a wavefront keeps the loads
 * in flight before it asks for the next: 1..3, 0 = all of them at once, -1 (the
 * default) = by size: all at once with 18-25 wavefronts per CU in small launches,
 * one or two from 16-96 MiB per input on (from 16 MiB with five and more inputs,
 * 32 MiB with three or four, 96 MiB with two), where 14-25 wavefronts per CU each
 * waiting for its previous input keep DRAM busier than bursts of all inputs.
 * Reduces of more than eight inputs (loaded eight at a time) take the settings of
 * nranks == 8; their defaults are two inputs in flight with 16 wavefronts per CU up
 * to 160 MiB per input and 14 above.
 * The settings belong to the calling thread: they shape the launches that thread
 * makes afterwards and nobody else's.  flagcxLocalInit checks once that the device
 * hands out LDS the way the caps assume (else no cap is applied). */
flagcxResult_t flagcxLocalTune(int nranks, int wavesPerCU);
flagcxResult_t flagcxLocalGetTune(int nranks, int *wavesPerCU);
flagcxResult_t flagcxLocalTuneLoads(int nranks, int inputsInFlight);
flagcxResult_t flagcxLocalGetTuneLoads(int nranks, int *inputsInFlight);

/* ------------------------------------------------------------------------- */
/* N-way elementwise reduction                                                */
/* ------------------------------------------------------------------------- */

/* recvbuff[i] = fold over j of sendbuffs[j][i], i in [0,count).
 *
 * The fold is the one the reference's host ring performs: acc = sendbuffs[0][i];
 * then for j = 1..nranks-1: acc = OP(sendbuffs[j][i], acc), where OP(a,b) is
 *   sum  a + b            (flagcx/service/utils.h:681-689)
 *   min  (b < a) ? b : a  (std::min(a,b), utils.h:691-699)
 *   max  (a < b) ? b : a  (std::max(a,b), utils.h:701-709)
 *   prod a * b, avg = sum then one division by nranks (the reference's host path
 *        rejects both, flagcx/service/bootstrap.cc:668-670; they exist here because
 *        the reduce-op enum carries them).
 * The call site replaced is `GENERATE_ALL_TYPES(datatype, sum, data_for_recv,
 * sendbuff + offset, data_for_recv, n)` (bootstrap.cc:649-671), i.e. op1 = the new
 * local input, op2 = the running partial, and on the device the vendor-CCL reduce
 * of flagcxC2cHomoFunc::run (flagcx/core/c2c_algo.cc:310-336).
 *
 * Integer sum/prod wrap modulo 2^bits.  fp16/bf16 sum, prod and avg accumulate in
 * fp32 and round to nearest even once; their min/max compare the widened values
 * and return the selected input bit pattern unchanged.  fp32/fp64 use their own
 * precision with no contraction or reassociation.  nranks == 1 is a copy
 * (bootstrap.cc:816-821).
 *
 * Errors: flagcxInvalidArgument for a NULL pointer, nranks outside
 * [1, FLAGCX_LOCAL_MAX_RANKS], an unknown datatype or op, a misaligned pointer or a
 * partial overlap; flagcxUnhandledDeviceError if the launch fails. */
flagcxResult_t flagcxLocalReduce(const void *const *sendbuffs, int nranks,
                                 void *recvbuff, size_t count,
                                 flagcxDataType_t datatype, flagcxRedOp_t op,
                                 flagcxStream_t stream);

/* What simulated rank `rank` ends with after the reference's ring reduce-scatter
 * with equal blocks (ReduceScatterBootstrap, flagcx/service/bootstrap.cc:848-874;
 * adaptor slot flagcxCCLAdaptor::reduceScatter, flagcx/adaptor/include/adaptor.h:118-121):
 * recvbuff[i] = fold of sendbuffs[r][rank*recvcount + i] taken in the ring's order
 * r = rank+1, rank+2, ..., rank (mod nranks) (bootstrap.cc:597-598,651-653).
 * recvbuff may equal sendbuffs[rank] + rank*recvcount (in place, flagcx.h:356). */
flagcxResult_t flagcxLocalReduceScatter(const void *const *sendbuffs, int nranks,
                                        int rank, void *recvbuff,
                                        size_t recvcount,
                                        flagcxDataType_t datatype,
                                        flagcxRedOp_t op, flagcxStream_t stream);

/* The same result produced chunk by chunk, the way the staging ring hands data
 * over (4 MiB steps, flagcx/core/p2p.cc:81-94): one launch per `chunkbytes` of
 * output.  chunkbytes == 0 selects FLAGCX_LOCAL_CHUNKSIZE; it must be a multiple of
 * the element size.  The chunks of one call do not depend on one another: from the
 * second on, a launch may start while its predecessor drains (the first still waits
 * for what the stream held before the call, and what follows the call for all of
 * them). */
flagcxResult_t flagcxLocalReduceScatterChunked(const void *const *sendbuffs,
                                               int nranks, int rank,
                                               void *recvbuff, size_t recvcount,
                                               flagcxDataType_t datatype,
                                               flagcxRedOp_t op,
                                               size_t chunkbytes,
                                               flagcxStream_t stream);

/* What every rank ends with after the reference's host ring all-reduce
 * (AllReduceBootstrap, flagcx/service/bootstrap.cc:810-827): the buffer is cut by
 * the chunk table of bootstrapRingAllReduce (bootstrap.cc:692-738) and chunk c is
 * folded in the order c+1, ..., c (mod nranks).  One recvbuff, since all ranks hold
 * the same bytes after the all-gather half.  recvbuff may equal one sendbuff. */
flagcxResult_t flagcxLocalAllReduce(const void *const *sendbuffs, int nranks,
                                    void *recvbuff, size_t count,
                                    flagcxDataType_t datatype, flagcxRedOp_t op,
                                    flagcxStream_t stream);

/* Several independent reductions that share nranks, datatype and op, enqueued in
 * as few launches as possible (one per 32 descriptors): the chunks of a pipelined
 * collective once they are all present, or ring chunks that differ in fold order.
 * Each descriptor is one flagcxLocalReduce.  Descriptors of one call run
 * concurrently: no descriptor's recvbuff may overlap another descriptor's buffers
 * (overlapping recvbuffs are rejected; inputs are the caller's responsibility). */
typedef struct {
  const void *const *sendbuffs; /* host array of nranks device pointers, fold order */
  void *recvbuff;
  size_t count;
} flagcxLocalReduceDesc;

flagcxResult_t flagcxLocalReduceBatch(const flagcxLocalReduceDesc *descs, int ndescs,
                                      int nranks, flagcxDataType_t datatype,
                                      flagcxRedOp_t op, flagcxStream_t stream);

/* A batch of sums over member lists of which `nzero` members are known to hold only
 * zeros and are not read: each descriptor lists the `nlive` members that hold data,
 * in fold order.  The result has the bytes that flagcxLocalReduceBatch gives over
 * the full lists with zero-filled buffers in the other places, wherever those stand:
 * for integers the sum of the members read; for floating-point types that sum plus
 * +0.0, added once before the rounding of the 16-bit types (zero members change a
 * sum in one way only: addends that are all -0.0 give +0.0).  This is the call
 * behind the fused replay of "clear all but the own slice, then all-reduce"
 * (flagcx/core/c2c_algo.cc:586-608 + 310-336).  nzero == 0 is
 * flagcxLocalReduceBatch; nzero > 0 with an op other than flagcxSum is
 * flagcxInvalidArgument. */
flagcxResult_t flagcxLocalReduceBatchSparse(const flagcxLocalReduceDesc *descs, int ndescs,
                                            int nlive, int nzero, flagcxDataType_t datatype,
                                            flagcxRedOp_t op, flagcxStream_t stream);

/* The same batch, launched BEFORE its inputs have arrived: the pipeline chunks of a
 * collective are known when it starts, only their arrival times are not.  Where the
 * reference's proxy would fold a chunk each time a receive completes (the loop
 * that such completions drive: flagcx/core/proxy.cc:1074-1182), the caller enqueues
 * the whole list once and then calls flagcxLocalGateOpen as chunks complete: the
 * wavefronts of descriptor i wait on the GPU, read nothing, until the gate's count
 * has passed i's number.  One ordinary launch per 32 descriptors, 3 to 4 % under
 * the rate of flagcxLocalReduceBatch, and a chunk's fold starts about 2 us after
 * its Open.
 * (An extension: the reference has no such entry point; its counterpart there is
 * that loop plus one collective call per completed chunk.)
 *
 * Descriptors get consecutive numbers per gate, from 0 at creation: this call's are
 * *first .. *first + ndescs - 1 (first may be NULL).  Open(upto) lets every
 * descriptor numbered below `upto` run; the count only rises, so chunks must be
 * opened in order (or as far as a contiguous prefix has arrived), and a count may
 * be opened before the launch that it belongs to.  Inputs must be complete in
 * device memory before their Open (an event or stream the caller has synchronised
 * with); results are read after the stream has been synchronised.
 * Restrictions (flagcxInvalidArgument otherwise): a non-NULL stream, nranks <= 8,
 * and within one descriptor every sendbuff agrees with recvbuff modulo 16 bytes.
 * Waiting wavefronts hold CU slots (up to half of every CU's) and most of the LDS:
 * a kernel that produces the inputs must not need the LDS they hold.
 * Work on another stream may be queued behind a launch that waits (streams share
 * hardware queues): never make an Open depend on the completion of such work.
 * The wait is bounded: when the count has not moved for
 * FLAGCX_FUNC_MAX_SPIN_COUNT polls (flagcxLocalSetMaxSpinCount; default 2^27,
 * minutes) the launch gives up, every wavefront that still waits leaves without
 * touching data, and the gate's state becomes 1 for good: later launches on it
 * are refused.  Create and Destroy allocate and synchronise (setup time);
 * Destroy abandons launches that still wait.  Open and Query touch pinned host
 * memory only and may be called from any thread.
 * A gate's count on the device lives in uncached memory, which wavefronts read
 * through the scalar path; with FLAGCX_LOCAL_GATE_CACHED=1 in the environment at
 * Create, or where the device gives no such memory, it lives in ordinary device
 * memory and is read with vector loads (same results, 2 to 8 % slower). */
typedef struct flagcxLocalGate *flagcxLocalGate_t;
#define FLAGCX_LOCAL_GATE_OK 0
#define FLAGCX_LOCAL_GATE_TIMED_OUT 1
flagcxResult_t flagcxLocalGateCreate(flagcxLocalGate_t *gate);
flagcxResult_t flagcxLocalGateDestroy(flagcxLocalGate_t gate);
flagcxResult_t flagcxLocalReduceBatchGated(flagcxLocalGate_t gate, const flagcxLocalReduceDesc *descs,
                                           int ndescs, int nranks, flagcxDataType_t datatype,
                                           flagcxRedOp_t op, flagcxStream_t stream, uint64_t *first);
flagcxResult_t flagcxLocalGateOpen(flagcxLocalGate_t gate, uint64_t upto);
/* A stream that belongs to the gate (valid until Destroy) and has a hardware queue that no
 * other stream is mapped to: a gated launch on it can hold up nothing else.  The runtime
 * spreads ordinary streams over a few hardware queues (four per process here), so with
 * more streams alive than that, the stream whose work completes the chunks may sit behind
 * the very launch that waits for them, which then ends in the spin bound.  Launch gated
 * batches here unless the caller controls how many streams the process holds.  It is a
 * blocking stream: NULL-stream work and the launch wait for each other. */
flagcxResult_t flagcxLocalGateOwnStream(flagcxLocalGate_t gate, flagcxStream_t *stream);
/* Descriptors numbered so far, the count, and the state (any pointer may be NULL). */
flagcxResult_t flagcxLocalGateQuery(flagcxLocalGate_t gate, uint64_t *launched, uint64_t *opened,
                                    int *state);

/* Consumer of the reference's reduce descriptor, which is declared but has no
 * producer or consumer there (flagcxReduceTrigger, flagcx/include/flagcx_kernel.h:30-35,
 * 52-73; host-producer API commented out at :96-98).  Same 256-bit layout:
 *   value[0] addr1, value[1] addr2, value[2] addr3,
 *   value[3] = count[0,32) | nthreads[32,48) | datatype[48,52) | redop[52,56) | reserved[63]
 * Meaning given here, after the host templates' (res, op1, op2) order
 * (flagcx/service/utils.h:681-709): addr3[i] = OP(addr1[i], addr2[i]), i < count;
 * nthreads is a hint and is ignored.  Triggers are executed in order; consecutive
 * triggers of the same datatype and op that do not depend on one another share a
 * launch. */
typedef struct {
#ifdef __cplusplus
  alignas(16)
#endif
  uint64_t value[4];
} flagcxLocalReduceTrigger;

static inline flagcxLocalReduceTrigger
flagcxLocalMakeReduceTrigger(const void *addr1, const void *addr2, void *addr3, uint32_t count,
                             uint32_t nthreads, flagcxDataType_t datatype, flagcxRedOp_t redop) {
  flagcxLocalReduceTrigger t;
  t.value[0] = (uint64_t)(uintptr_t)addr1;
  t.value[1] = (uint64_t)(uintptr_t)addr2;
  t.value[2] = (uint64_t)(uintptr_t)addr3;
  t.value[3] = (uint64_t)count | ((uint64_t)(nthreads & 0xffffu) << 32) |
               ((uint64_t)((unsigned)datatype & 0xfu) << 48) | ((uint64_t)((unsigned)redop & 0xfu) << 52);
  return t;
}

flagcxResult_t flagcxLocalReduceTriggers(const flagcxLocalReduceTrigger *triggers, int ntriggers,
                                         flagcxStream_t stream);

/* The chunk table itself (bootstrap.cc:692-738): offsets[i], lengths[i] in bytes
 * for i in [0,nranks).  Host-only. */
flagcxResult_t flagcxLocalRingChunkTable(size_t count, flagcxDataType_t datatype,
                                         int nranks, size_t *offsets,
                                         size_t *lengths);

/* ------------------------------------------------------------------------- */
/* Chunk copy / zero-fill / pack / unpack                                      */
/* ------------------------------------------------------------------------- */

/* Device-to-device byte copy on the stream; replaces the deviceMemcpy(D2D) of
 * the staging loops (flagcx/core/p2p.cc:86-89,182-185,245-247;
 * flagcx/core/net.cc:153-161,298-306; hip_adaptor.cc:16-29).  Buffers must not
 * overlap unless dst == src. */
flagcxResult_t flagcxLocalMemcpy(void *dst, const void *src, size_t size,
                                 flagcxStream_t stream);

/* Byte fill; replaces deviceMemset (hip_adaptor.cc:31-41). */
flagcxResult_t flagcxLocalMemset(void *ptr, int value, size_t size,
                                 flagcxStream_t stream);

/* flagcxC2cRefreshFunc::run (flagcx/core/c2c_algo.cc:586-608) in one launch: when
 * op == flagcxSum, zero elements [start, start+offset) and
 * [start+offset+count, start+totalcount) of buff and leave [start+offset,
 * start+offset+count) alone; any other op does nothing.  offset+count >
 * totalcount is flagcxInvalidArgument. */
flagcxResult_t flagcxLocalRefresh(void *buff, size_t start, size_t offset,
                                  size_t count, size_t totalcount,
                                  flagcxDataType_t datatype, flagcxRedOp_t op,
                                  flagcxStream_t stream);

/* Strided gather: dst[c*chunkbytes + b] = src[c*srcstride + b] for c in
 * [0,nchunks), b in [0,chunkbytes); srcstride >= chunkbytes.  Rank r's chunk at
 * buffer + r*stride is the addressing of flagcx/adaptor/ccl/rccl_adaptor.cc:103-159. */
flagcxResult_t flagcxLocalPack(void *dst, const void *src, size_t nchunks,
                               size_t chunkbytes, size_t srcstride,
                               flagcxStream_t stream);

/* Strided scatter, the inverse: dst[c*dststride + b] = src[c*chunkbytes + b].
 * Bytes of dst between chunks are not written. */
flagcxResult_t flagcxLocalUnpack(void *dst, const void *src, size_t nchunks,
                                 size_t chunkbytes, size_t dststride,
                                 flagcxStream_t stream);

/* Flatten n separate device buffers of `bytes` each into one contiguous buffer
 * (dst + j*bytes), one launch instead of the per-tensor copy_ loop of
 * plugin/torch/flagcx/src/backend_flagcx.cpp:831-840,942-951.  srcs is a host
 * array, n <= FLAGCX_LOCAL_MAX_RANKS. */
flagcxResult_t flagcxLocalPackList(void *dst, const void *const *srcs, int n,
                                   size_t bytes, flagcxStream_t stream);

/* The inverse (backend_flagcx.cpp:429-445,753-769). */
flagcxResult_t flagcxLocalUnpackList(void *const *dsts, const void *src, int n,
                                     size_t bytes, flagcxStream_t stream);

/* One source copied to several destinations, and several such copies in one call: what a
 * broadcast (flagcxC2cHomoFunc::run, flagcx/core/c2c_algo.cc:464-472 ->
 * flagcx/adaptor/ccl/rccl_adaptor.cc:161-168) or an all-gather (c2c_algo.cc:337-345 ->
 * rccl_adaptor.cc:188-195) moves when the ranks of a cluster are buffers on one GPU.
 * Destinations that agree with their source modulo 16 bytes share one read of it: the
 * launch moves (1 + ndsts) * bytes instead of 2 * ndsts * bytes; the others are plain
 * copies.  A destination equal to its source is skipped (the root of an in-place
 * broadcast).  The copies of one call run concurrently: a destination that overlaps any
 * other buffer of the call -> flagcxInvalidArgument, before anything is launched.
 * dsts is a host array. */
#define FLAGCX_LOCAL_FANOUT_MAX 64       /* copies per call */
#define FLAGCX_LOCAL_FANOUT_MAX_DSTS 256 /* destinations per call, all copies together */
typedef struct {
  const void *src;
  void *const *dsts;
  int ndsts;
  size_t bytes;
} flagcxLocalFanoutDesc;
flagcxResult_t flagcxLocalCopyFanout(const flagcxLocalFanoutDesc *descs, int ndescs,
                                     flagcxStream_t stream);

/* ------------------------------------------------------------------------- */
/* Device-producer / host-consumer trigger FIFO                                */
/* ------------------------------------------------------------------------- */
/* The reference's kernel FIFO (flagcx/include/flagcx_kernel.h:7-49,75-88): a pinned
 * host buffer of 64-bit words [capacity, consumed, produced, entries...]; an entry
 * is {fst, snd} with fst = address and
 * snd = count[0,32) | peerRank[32,52) | datatype[52,56) | prim[56,60). */
#define FLAGCX_LOCAL_FIFO_CAPACITY 16 /* FLAGCX_KERNEL_FIFO_CAPACITY */
#define FLAGCX_LOCAL_PRIM_SEND 0      /* flagcxDevicePrimSend .. Wait, flagcx_kernel.h:9-14 */
#define FLAGCX_LOCAL_PRIM_RECV 1
#define FLAGCX_LOCAL_PRIM_TERM 2
#define FLAGCX_LOCAL_PRIM_WAIT 3

typedef struct {
  uint64_t fst;
  uint64_t snd;
} flagcxLocalDeviceTrigger;

/* Getters of flagcxDeviceTrigger (flagcx/core/flagcx_kernel_host.cc:9-29). */
static inline uint64_t flagcxLocalTriggerAddr(const flagcxLocalDeviceTrigger *t) { return t->fst; }
static inline uint64_t flagcxLocalTriggerCount(const flagcxLocalDeviceTrigger *t) { return t->snd & 0xffffffffull; }
static inline uint64_t flagcxLocalTriggerPeerRank(const flagcxLocalDeviceTrigger *t) { return (t->snd >> 32) & 0xfffffull; }
static inline uint64_t flagcxLocalTriggerDatatype(const flagcxLocalDeviceTrigger *t) { return (t->snd >> 52) & 0xfull; }
static inline uint64_t flagcxLocalTriggerType(const flagcxLocalDeviceTrigger *t) { return (t->snd >> 56) & 0xfull; }

/* flagcxFifo::flagcxFifoInit / flagcxFifoDestroy (flagcx_kernel_host.cc:31-50):
 * allocates (setup time, not the hot path) and frees the pinned buffer. */
flagcxResult_t flagcxLocalFifoInit(void **fifoBuffer);
flagcxResult_t flagcxLocalFifoDestroy(void *fifoBuffer);
/* Host side: dequeue (flagcx_kernel_host.cc:52-73).  An empty queue yields a zero
 * trigger and flagcxSuccess. */
flagcxResult_t flagcxLocalFifoDequeue(void *fifoBuffer, flagcxLocalDeviceTrigger *trigger);
/* flagcxP2pDemo (flagcx/kernels/device_collective_demo.cu:27-34): one lane enqueues
 * Send, Recv, Term and Wait triggers, then waits until the host has drained the
 * queue.  All device-side waits give up after the spin bound of deviceAsyncLoad. */
flagcxResult_t flagcxLocalP2pDemo(const void *sendbuff, void *recvbuff, size_t count,
                                  flagcxDataType_t datatype, int sendPeer, int recvPeer,
                                  void *fifoBuffer, flagcxStream_t stream);

/* ------------------------------------------------------------------------- */
/* Host-producer / device-consumer reduce queue                                */
/* ------------------------------------------------------------------------- */
/* The other direction of the kernel FIFO, which the reference declares for
 * flagcxReduceTrigger and leaves commented out
 * (`enqueue(flagcxReduceTrigger)` on the host, `dequeue` on the device,
 * flagcx/include/flagcx_kernel.h:96-98): the host appends reduce descriptors to a
 * pinned ring [capacity, consumed, produced, ...] and ONE resident kernel folds
 * them as they arrive, so a 4 MiB chunk costs no kernel launch.  The queue owns a
 * non-blocking stream for that kernel, as the kernel proxy owns its stream
 * (flagcx/core/proxy.cc:1094-1097).
 *
 * A queue is created for one element type and one op; entries carry 1..maxRanks
 * (at most 8) inputs.  The result is that of running the entries one after
 * another: independent entries are folded concurrently, and an entry that reads or
 * overwrites what an earlier entry still in flight writes (or overwrites what it
 * reads) is held back until everything before it has finished.
 * The producer appends an entry only when its inputs are complete in device
 * memory (an event or stream it has synchronised with), and reads results after
 * Wait(ticket) or Stop.  Create / Start / Stop / Destroy allocate or synchronise
 * (setup time); Enqueue, Query and Wait touch pinned host memory only.
 *
 * While the consumer is on the GPU it holds up to half of every CU's wavefront
 * slots and four fifths of its LDS: other launches run next to it, more slowly,
 * except those on streams that the runtime has mapped to the same hardware queue,
 * which wait like behind any other kernel.  So the consumer does not outstay its
 * work: after `linger` polls (about 3 us each, default 64) with nothing
 * outstanding it parks, i.e. the kernel ends, and the next Enqueue launches it
 * again (about 20 us more for that entry).  Device-wide synchronisation
 * (hipDeviceSynchronize, hipFree) therefore returns once the queue has drained
 * and lingered.  With linger 0 the consumer stays until Stop.  If entries are
 * outstanding and nothing moves for FLAGCX_FUNC_MAX_SPIN_COUNT polls
 * (flagcxLocalSetMaxSpinCount; default 2^27, minutes) the consumer gives up,
 * state 3. */
typedef struct flagcxLocalReduceFifo *flagcxLocalReduceFifo_t;
#define FLAGCX_LOCAL_REDUCE_FIFO_IDLE 0
#define FLAGCX_LOCAL_REDUCE_FIFO_RUNNING 1
#define FLAGCX_LOCAL_REDUCE_FIFO_STOPPED 2
#define FLAGCX_LOCAL_REDUCE_FIFO_TIMED_OUT 3
#define FLAGCX_LOCAL_REDUCE_FIFO_PARKED 4 /* started, idle, off the GPU until the next entry */

flagcxResult_t flagcxLocalReduceFifoCreate(flagcxLocalReduceFifo_t *fifo, int capacity, int maxRanks,
                                           flagcxDataType_t datatype, flagcxRedOp_t op);
/* Stop (if running), then free everything. */
flagcxResult_t flagcxLocalReduceFifoDestroy(flagcxLocalReduceFifo_t fifo);
/* Launches the consumer; counters restart at zero.  A stopped or timed-out queue
 * can be started again. */
flagcxResult_t flagcxLocalReduceFifoStart(flagcxLocalReduceFifo_t fifo);
/* Appends a stop entry behind everything enqueued so far and waits until the
 * consumer has finished those entries and left the GPU. */
flagcxResult_t flagcxLocalReduceFifoStop(flagcxLocalReduceFifo_t fifo);
/* Host `enqueue(flagcxReduceTrigger)`: addr3 = OP(addr1, addr2) over `count`
 * elements, as flagcxLocalReduceTriggers; the trigger's datatype and redop must be
 * the queue's.  *ticket (may be NULL) is the value `consumed` reaches when this
 * entry is done.  flagcxInProgress: the ring is full, try again. */
flagcxResult_t flagcxLocalReduceFifoEnqueue(flagcxLocalReduceFifo_t fifo, const flagcxLocalReduceTrigger *trigger,
                                            uint64_t *ticket);
/* The N-way form: recvbuff = fold of sendbuffs[0..nranks) in array order, as
 * flagcxLocalReduce, nranks <= maxRanks. */
flagcxResult_t flagcxLocalReduceFifoEnqueueReduce(flagcxLocalReduceFifo_t fifo, const void *const *sendbuffs,
                                                  int nranks, void *recvbuff, size_t count, uint64_t *ticket);
/* Counters and state (any pointer may be NULL); never blocks. */
flagcxResult_t flagcxLocalReduceFifoQuery(flagcxLocalReduceFifo_t fifo, uint64_t *produced, uint64_t *consumed,
                                          int *state);
/* Spins on the host until consumed >= ticket.  flagcxInvalidArgument if the ticket
 * has not been handed out; an error if the consumer exits first. */
flagcxResult_t flagcxLocalReduceFifoWait(flagcxLocalReduceFifo_t fifo, uint64_t ticket);
/* Resident wavefronts per CU of the next Start (1..16; the default depends on
 * maxRanks).  Not between Start and Stop. */
flagcxResult_t flagcxLocalReduceFifoSetWaves(flagcxLocalReduceFifo_t fifo, int wavesPerCU);
/* What the queue was created for (any pointer may be NULL). */
flagcxResult_t flagcxLocalReduceFifoGetType(flagcxLocalReduceFifo_t fifo, flagcxDataType_t *datatype,
                                            flagcxRedOp_t *op, int *maxRanks);
/* Traffic, (nranks + 1) * bytes per entry, of the entries the consumer works on
 * together beyond the oldest unfinished one (default 256 MiB, measured best: a
 * narrow window keeps the wavefronts on neighbouring tiles and inside the
 * last-level cache; two entries may always be in work).  Not between Start and Stop. */
flagcxResult_t flagcxLocalReduceFifoSetWindow(flagcxLocalReduceFifo_t fifo, size_t bytes);
/* Idle polls before the consumer parks (0: never).  Not between Start and Stop. */
flagcxResult_t flagcxLocalReduceFifoSetLinger(flagcxLocalReduceFifo_t fifo, int64_t polls);
/* own != 0: the consumer gets a hardware queue that no other stream is mapped to, so that
 * no launch on any stream ever waits behind it (the runtime spreads ordinary streams over a
 * few hardware queues, four per process here, and work on a stream that lands on the
 * consumer's waits until the consumer parks).  The price: such a stream is a blocking one,
 * i.e. work on the NULL stream and the consumer wait for each other.  For callers that
 * keep their work on non-blocking streams of their own, as the reference's proxies do
 * (flagcx/core/proxy.cc:1094-1097); leave it off where the NULL stream is in use (PyTorch's
 * default stream is).  Default off.  Not between Start and Stop. */
flagcxResult_t flagcxLocalReduceFifoSetOwnQueue(flagcxLocalReduceFifo_t fifo, int own);
/* Workgroups (one wavefront each) of the running consumer: 1 leader + workers. */
flagcxResult_t flagcxLocalReduceFifoGetGrid(flagcxLocalReduceFifo_t fifo, unsigned *workgroups);
const char *flagcxLocalReduceFifoGetLastError(flagcxLocalReduceFifo_t fifo);

/* ------------------------------------------------------------------------- */
/* Staging ring (the pipeline either side of the reduce)                       */
/* ------------------------------------------------------------------------- */
/* The 16 x 4 MiB staging ring of the reference's proxies
 * (FLAGCX_P2P_STEPS x FLAGCX_P2P_CHUNKSIZE, flagcx/core/p2p.h:11-15;
 * MAXSTEPS x CHUNKSIZE, flagcx/core/net.h:19-22) on one GPU: a producer stream
 * copies chunk `step` into slot step % steps like flagcxP2pProxySend
 * (flagcx/core/p2p.cc:75-107), a consumer stream takes it out like
 * flagcxP2pProxyRecv (p2p.cc:170-205); sendHead / recvTail are one "filled" and
 * one "freed" event per slot.  ringBuffer is the caller's device memory of at
 * least steps * npeers * chunkBytes bytes (0 selects 4 MiB / 16); Create
 * allocates events only.  Calls on one ring must not overlap. */
typedef struct flagcxLocalRing *flagcxLocalRing_t;
flagcxResult_t flagcxLocalRingCreate(flagcxLocalRing_t *ring, void *ringBuffer, size_t ringBytes,
                                     int npeers, size_t chunkBytes, int steps);
flagcxResult_t flagcxLocalRingDestroy(flagcxLocalRing_t ring);
/* One message src -> ring -> dst in chunk steps (send/recv staging).  Work is
 * enqueued on copyStream (producer) and stream (consumer); the result is complete
 * when `stream` is.  Neither stream may be NULL. */
flagcxResult_t flagcxLocalRingSendRecv(flagcxLocalRing_t ring, void *dst, const void *src, size_t size,
                                       flagcxStream_t copyStream, flagcxStream_t stream);
/* flagcxLocalReduceScatter with the nranks-1 peers' slices arriving through the
 * ring: per chunk one launch stages all peers' pieces into the slot and one
 * reduce folds them with the local piece into recvbuff, so the reduce of chunk i
 * overlaps the staging of chunk i+1.  Same bytes as flagcxLocalReduceScatter. */
flagcxResult_t flagcxLocalRingReduceScatter(flagcxLocalRing_t ring, const void *const *sendbuffs,
                                            int nranks, int rank, void *recvbuff, size_t recvcount,
                                            flagcxDataType_t datatype, flagcxRedOp_t op,
                                            flagcxStream_t copyStream, flagcxStream_t stream);
/* The same shard driven the way the reference's proxy thread drives its steps
 * (flagcx/core/p2p.cc:75-107,170-205): the caller's thread issues each step's
 * staging copy on copyStream, records an event, polls it (eventQuery) and then
 * hands the step to a running reduce queue; a slot is reused when that entry's
 * ticket is consumed.  No stream waits for another and no reduce is launched.
 * Type and op are the queue's; nranks <= its maxRanks.  Inputs must be complete
 * in copyStream's order.  Blocks until recvbuff is complete. */
flagcxResult_t flagcxLocalRingReduceScatterFifo(flagcxLocalRing_t ring, flagcxLocalReduceFifo_t fifo,
                                                const void *const *sendbuffs, int nranks, int rank,
                                                void *recvbuff, size_t recvcount, flagcxStream_t copyStream);

/* No counterpart in the reference: this entry point exists for callers that cannot
 * allocate - code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc - and so can neither create a ring (events) nor bring a ring
 * buffer.  It is flagcxLocalRingReduceScatter on ONE stream with the staging slots
 * in a fixed area inside the library's own device image
 * (FLAGCX_LOCAL_STATIC_STAGING_BYTES per GPU, held from the moment the library's
 * code is loaded on that GPU until the process ends): one launch stages the
 * nranks-1 peers' slices of shard `rank` there, one reduce folds them with the
 * local slice into recvbuff, in the ring's order rank+1, ..., rank - the same
 * bytes as flagcxLocalRingReduceScatter and flagcxLocalReduceScatter.  Calls no
 * hipMalloc / hipFree and creates no stream or event.
 * Limit: (nranks - 1) * roundUp(recvcount * elementSize + (recvbuff mod 128), 256)
 * <= FLAGCX_LOCAL_STATIC_STAGING_BYTES, else flagcxInvalidArgument (a staged slice
 * sits as far into its 128-byte line as recvbuff does into its own).  Every call on
 * a GPU uses that GPU's one staging area: calls on one stream follow one another;
 * calls that overlap in time on different streams of one GPU race on it. */
#define FLAGCX_LOCAL_STATIC_STAGING_BYTES (8ULL * 1024 * 1024)
flagcxResult_t flagcxLocalStagedReduceScatterNoAlloc(const void *const *sendbuffs, int nranks, int rank,
                                                     void *recvbuff, size_t recvcount,
                                                     flagcxDataType_t datatype, flagcxRedOp_t op,
                                                     flagcxStream_t stream);

/* ------------------------------------------------------------------------- */
/* C2C plan replay on one GPU                                                  */
/* ------------------------------------------------------------------------- */
/* Replays, for ALL simulated ranks in lock step, the per-rank plans that
 * flagcxC2cPlanner exports and imports as XML (flagcx/core/c2c_algo.cc:973-1087,
 * format in flagcx/core/c2c_ir.h:62-176), stage by stage as
 * flagcxC2cPlanner::execute does (c2c_algo.cc:2142-2290).  Homo functions
 * (flagcxC2cHomoFunc::run, c2c_algo.cc:286-511) run on the ranks of a cluster
 * (homoType 1: on its inter-ranks) with the local reduce / copy kernels in place
 * of the vendor CCL, folding in homo-rank order; Send / Recv homo functions of all
 * three homoTypes and hetero P2P ops become device copies between the ranks'
 * buffers; the refresh function is flagcxLocalRefresh.  `root` of Execute is a
 * global rank and reaches the homo functions as its rank inside its cluster, like
 * globalrank2homorank[root] (c2c_algo.cc:2147,2170).  An AlltoAllv plan takes its
 * counts and displacements, which are call arguments and not part of a plan, from
 * flagcxLocalPlanSetAlltoAllv; a document with negative offsets or counts is
 * flagcxInvalidArgument at import.  Every rank walks its own step tables, as in the
 * reference: a rank whose table for a step is shorter than its peers' takes no part
 * in their later functions of that step (c2c_algo.cc:2177,2204,2247,2277), and a
 * collective that then lacks a member is flagcxInvalidUsage where the reference
 * would hang.
 * commOp 12 (LocCpy) and 13 (LocRed), reserved by the reference's plan DSL
 * (flagcx/tools/utils.py:43-44), are rank-local copy and
 * recv = OP(send, recv).  Host-side errors of a plan are reported through
 * flagcxLocalPlanGetLastError.  A plan object belongs to one thread at a time (its
 * error text and traffic figures are per object); different plans may be used from
 * different threads at once. */
typedef struct flagcxLocalPlan *flagcxLocalPlan_t;

/* clusterIds[r]: cluster of global rank r (0-based, dense).  isInterRank[r] != 0:
 * rank r is one of its cluster's inter-ranks (NULL: every rank is).  totalCount:
 * elements of the collective (send or recv count, as flagcxC2cPlanner's
 * totalCount_).  redOp other than sum/max/min is flagcxNotSupported at execute,
 * like c2c_algo.cc:2047-2053. */
flagcxResult_t flagcxLocalPlanCreate(flagcxLocalPlan_t *plan, int nranks, const int *clusterIds,
                                     const int *isInterRank, size_t totalCount,
                                     flagcxCommOp_t commOp, flagcxRedOp_t redOp);
flagcxResult_t flagcxLocalPlanDestroy(flagcxLocalPlan_t plan);
/* Reads / writes <prefix>_<rank>.xml for every rank. */
flagcxResult_t flagcxLocalPlanImportXml(flagcxLocalPlan_t plan, const char *prefix);
flagcxResult_t flagcxLocalPlanExportXml(flagcxLocalPlan_t plan, const char *prefix);
/* Number of chunks of plan documents that carry no <nChunks> (those written by the
 * reference's plan DSL, flagcx/tools/algorithm.py:160-181; exportXml always writes
 * it, c2c_algo.cc:1058): a document's offsets and counts are in units of
 * totalCount / nChunks elements.  Call before ImportXml. */
flagcxResult_t flagcxLocalPlanSetChunks(flagcxLocalPlan_t plan, size_t nchunks);
/* Counts and displacements of an AlltoAllv, in elements: four nranks x nranks
 * matrices, row r = the arrays rank r passes to flagcxC2cPlanner::execute
 * (flagcx/core/c2c_algo.cc:2042-2046; NULL -> flagcxInvalidArgument as
 * c2c_algo.cc:2083-2089).  The plan's hetero functions carry the cross-cluster
 * pieces (c2c_algo.cc:1618-1630); its AlltoAllv homo function moves the pieces
 * inside a cluster from these arrays (c2c_algo.cc:482-508).  Call before Execute. */
flagcxResult_t flagcxLocalPlanSetAlltoAllv(flagcxLocalPlan_t plan, const size_t *sendCounts,
                                           const size_t *sDispls, const size_t *recvCounts,
                                           const size_t *rDispls);
/* 0 sequential, 1 pipeline, 2 input (default after import). */
flagcxResult_t flagcxLocalPlanSetAlgorithm(flagcxLocalPlan_t plan, int algorithm);
/* How the refresh function and the sums behind it are replayed.  The reference
 * assembles a sum across a cluster by clearing, in every member's buffer, all but
 * the member's own slice (flagcxC2cRefreshFunc::run, c2c_algo.cc:586-608) and then
 * reducing the whole buffers with the vendor CCL (c2c_algo.cc:310-336), which reads
 * the zeros back.
 *   fused = 1 (default): a refresh only records the ranges it clears; copies out of
 *     such a range move the record, a write ends it, a sum reads only the members
 *     whose slice holds data (flagcxLocalReduceBatchSparse) and what is still
 *     recorded for a receive buffer when the plan ends is written then.  Ranges in a
 *     scratch buffer that the reference allocates for the call and frees at its end
 *     (c2c_algo.cc:2122-2129,2292-2295) are never written.
 *   fused = 0: every refresh is a zero-fill (flagcxLocalRefresh) and every
 *     collective reads all of its members, as the reference does.
 * Every receive buffer ends with the same bytes either way, signed zeros included. */
flagcxResult_t flagcxLocalPlanSetFused(flagcxLocalPlan_t plan, int fused);
/* Algorithmic bytes (2 per copied byte, (k + 1) * count * size per k-input
 * reduction, 1 per cleared byte) and kernel launches of the last Execute. */
flagcxResult_t flagcxLocalPlanGetTraffic(flagcxLocalPlan_t plan, uint64_t *bytes, uint64_t *launches);
/* Host arrays of one device pointer per rank.  Scratch is used where the reference
 * allocates one for the call - every rank of a ReduceScatter or Scatter, the
 * non-root ranks of a Gather (c2c_algo.cc:2121-2129): there hetero receives and a
 * refresh of buffType -1 go to scratchbuffs[rank], which must not be NULL; on every
 * other rank they go to recvbuffs[rank] (c2c_algo.cc:2131,2157-2158) and the scratch
 * pointer, which may be NULL, is only what functions that name scratch explicitly
 * (sendType / recvType / buffType 2) get.  No buffer is taken to hold more than
 * totalCount elements (c2c_algo.cc:623,2124): a function or refresh that reaches past
 * that returns flagcxInvalidArgument before it is launched (what was enqueued ahead of
 * it still runs).  Enqueues everything on `stream`. */
flagcxResult_t flagcxLocalPlanExecute(flagcxLocalPlan_t plan, const void *const *sendbuffs,
                                      void *const *recvbuffs, void *const *scratchbuffs,
                                      flagcxDataType_t datatype, int root, flagcxStream_t stream);
const char *flagcxLocalPlanGetLastError(flagcxLocalPlan_t plan);

/* ------------------------------------------------------------------------- */
/* Launcher-convention symbols                                                */
/* ------------------------------------------------------------------------- */
/* These have the reference's device-function shape
 *   typedef void (*flagcxLaunchFunc_t)(flagcxStream_t, void *)
 * (flagcx/adaptor/include/adaptor.h:15) so that loadKernelSymbol
 * (flagcx/core/launch_kernel.cc:11-29) can dlsym them from the library named by
 * FLAGCX_DEVICE_FUNC_PATH (flagcx/flagcx.cc:552-562) and launchDeviceFunc
 * (hip_adaptor.cc:263-269) can call them.  They return nothing, so the result
 * code is written into the argument block. */

typedef struct {
  const void *const *sendbuffs; /* host array of nranks device pointers */
  void *recvbuff;
  uint64_t count;
  int32_t nranks;
  int32_t datatype; /* flagcxDataType_t */
  int32_t op;       /* flagcxRedOp_t */
  int32_t result;   /* out: flagcxResult_t */
} flagcxLocalReduceArgs;

typedef struct {
  void *dst;
  const void *src;
  uint64_t size;
  int32_t result; /* out */
  int32_t reserved;
} flagcxLocalCopyArgs;

void flagcxLocalReduceFunc(flagcxStream_t stream, void *args /* flagcxLocalReduceArgs* */);
void flagcxLocalCopyFunc(flagcxStream_t stream, void *args /* flagcxLocalCopyArgs* */);

/* The two symbols flagcxCommInitRank resolves from FLAGCX_DEVICE_FUNC_PATH
 * (flagcx/flagcx.cc:552-562); gfx950 versions of
 * flagcx/kernels/device_async_kernel.dev:14-23.  args is a device bool*:
 * Store sets it; Load returns once it is set or after the spin bound
 * (FLAGCX_FUNC_MAX_SPIN_COUNT polls, default 2^27) - the reference spins without
 * bound.  These keep the reference's un-prefixed names because it looks them up
 * by name. */
void deviceAsyncStore(flagcxStream_t stream, void *args /* bool* on the device */);
void deviceAsyncLoad(flagcxStream_t stream, void *args /* bool* on the device */);
/* Overrides the spin bound of deviceAsyncLoad (negative: back to the environment). */
void flagcxLocalSetMaxSpinCount(int64_t polls);

#ifdef __cplusplus
}
#endif
#endif /* FLAGCX_AMD_H_ */
