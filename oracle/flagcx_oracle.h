/*
 * flagcx_oracle.h - CPU restatement of the reference's host-side reduce path.
 *
 * TEST INFRASTRUCTURE ONLY.  This code is the checker for the HIP library: only
 * tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may load
 * it.  Nothing under flagcx_amd/ links, imports or calls it.
 *
 * Each function names the reference lines it follows.  Pinning status:
 *   - binary sum/min/max on the eight reference dtypes: pinned against the
 *     reference's own templates compiled from /root/reference (oracle/_ref) and
 *     against golden vectors generated from them (tests/golden).
 *   - ring fold order, chunk table, refresh ranges, type sizes: pinned by closed
 *     forms / brute force and the reference's own test patterns (i % 10).
 *   - fp16 / bf16 conversion and accumulation, prod, avg: the reference rejects
 *     them on the host path (flagcx/service/utils.h:674-678,
 *     flagcx/service/bootstrap.cc:668-670); pinned against numpy float16 /
 *     torch bfloat16 library arithmetic and exact small-integer cases.
 *   - what the vendor CCL does on the device path (rounding and fold order
 *     inside RCCL, reached from flagcx/core/c2c_algo.cc:310-336): parity unpinned.
 */
#ifndef FLAGCX_ORACLE_H_
#define FLAGCX_ORACLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* flagcx/flagcx.cc:30-61 */
size_t oracle_type_size(int dtype);

/* flagcx/service/utils.h:648-709 + flagcx/service/bootstrap.cc:649-671.
 * res[i] = OP(op1[i], op2[i]); res may alias op1 or op2.
 * strict != 0: behave exactly like the reference host path, i.e. return
 * flagcxInvalidArgument (4) for fp16, bf16, unknown dtypes, prod, avg.
 * strict == 0: also accept the extensions defined in include/flagcx_amd.h
 * (prod; fp16/bf16 computed in fp32 and rounded once per call; avg is not a
 * binary op and stays invalid here). */
int oracle_binary(int op, int dtype, void *res, const void *op1, const void *op2,
                  size_t n, int strict);

/* N-way fold in array order: acc = srcs[0]; acc = OP(srcs[j], acc), j=1..k-1.
 * fp16/bf16 sum/prod/avg keep acc in fp32 and round once at the end.
 * avg divides the fold-sum by k once.  Returns 0 or flagcxInvalidArgument. */
int oracle_reduce(const void *const *srcs, int k, void *dst, size_t n, int dtype,
                  int op);

/* Whole-job simulation of bootstrapRingReduceScatter
 * (flagcx/service/bootstrap.cc:569-690) for all nranks at once, sockets replaced
 * by memcpy between the simulated ranks' temp buffers.  sendbuffs[r] is rank r's
 * send buffer, recvbuffs[r] receives length[r] bytes.  strict as above; in
 * non-strict mode half types and prod/avg are evaluated through oracle_reduce in
 * the ring's order. */
int oracle_ring_reduce_scatter(const void *const *sendbuffs, void *const *recvbuffs,
                               int nranks, const size_t *offset,
                               const size_t *length, int dtype, int op,
                               int strict);

/* flagcx/service/bootstrap.cc:692-738 */
void oracle_ring_chunk_table(size_t size_bytes, size_t type_size, int nranks,
                             size_t *offset, size_t *length);

/* bootstrapRingAllReduce (bootstrap.cc:702-749) incl. the nranks==1 shortcut of
 * AllReduceBootstrap (:816-821): chunk table, ring reduce-scatter, all-gather.
 * recvbuff receives the bytes every rank ends with. */
int oracle_ring_allreduce(const void *const *sendbuffs, void *recvbuff, int nranks,
                          size_t count, int dtype, int op, int strict);

/* ReduceScatterBootstrap (bootstrap.cc:848-874) for one rank. */
int oracle_reduce_scatter_rank(const void *const *sendbuffs, void *recvbuff,
                               int nranks, int rank, size_t recvcount, int dtype,
                               int op, int strict);

/* flagcxC2cRefreshFunc::run (flagcx/core/c2c_algo.cc:586-608) on host memory. */
void oracle_refresh(void *buff, size_t start, size_t offset, size_t count,
                    size_t totalcount, size_t type_size, int op);

/* byte movers */
void oracle_pack(void *dst, const void *src, size_t nchunks, size_t chunkbytes,
                 size_t srcstride);
void oracle_unpack(void *dst, const void *src, size_t nchunks, size_t chunkbytes,
                   size_t dststride);

/* conversions (round to nearest even on narrowing) */
float oracle_half_to_float(uint16_t h);
uint16_t oracle_float_to_half(float f);
float oracle_bf16_to_float(uint16_t b);
uint16_t oracle_float_to_bf16(float f);

/* Timing helper for the CPU baseline: runs oracle_reduce `iters` times on nthreads
 * threads (thread t reduces its own contiguous 1/nthreads share, one simulated
 * rank each) and returns the median wall seconds per iteration.
 * clock_gettime(CLOCK_MONOTONIC) like clockNano (flagcx/service/utils.h:60-64). */
double oracle_time_reduce(const void *const *srcs, int k, void *dst, size_t n,
                          int dtype, int op, int nthreads, int warmup, int iters);

#ifdef __cplusplus
}
#endif
#endif
