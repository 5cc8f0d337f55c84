/*
 * flagcx_oracle.c - CPU restatement of the reference's host-side reduce path.
 * TEST INFRASTRUCTURE ONLY; see flagcx_oracle.h for who may use it and for the
 * pinning status of each function.
 */
#define _GNU_SOURCE
#include "flagcx_oracle.h"

#include <pthread.h>
#include <stdlib.h>
#include <string.h>
#include <time.h>

enum { R_OK = 0, R_INVALID = 4 };
enum { T_I8 = 0, T_U8, T_I32, T_U32, T_I64, T_U64, T_F16, T_F32, T_F64, T_BF16 };
enum { OP_SUM = 0, OP_PROD, OP_MAX, OP_MIN, OP_AVG };

/* flagcx/flagcx.cc:30-61: 1,1,4,4,8,8,2,4,8,2 and 0 for anything else */
size_t oracle_type_size(int dtype) {
  switch (dtype) {
    case T_I8: case T_U8: return 1;
    case T_I32: case T_U32: case T_F32: return 4;
    case T_I64: case T_U64: case T_F64: return 8;
    case T_F16: case T_BF16: return 2;
    default: return 0;
  }
}

/* ---------------------------------------------------------------- halves */

float oracle_half_to_float(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1fu;
  uint32_t man = h & 0x3ffu;
  uint32_t out;
  if (exp == 0) {
    if (man == 0) {
      out = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do { man <<= 1; e++; } while (!(man & 0x400u));
      out = sign | ((uint32_t)(127 - 15 - e) << 23) | ((man & 0x3ffu) << 13);
    }
  } else if (exp == 31) {
    out = sign | 0x7f800000u | (man << 13);
  } else {
    out = sign | ((exp + 127 - 15) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &out, 4);
  return f;
}

uint16_t oracle_float_to_half(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint16_t sign = (uint16_t)((x >> 16) & 0x8000u);
  uint32_t ax = x & 0x7fffffffu;
  if (ax >= 0x7f800000u) { /* inf / nan */
    if (ax == 0x7f800000u) return sign | 0x7c00u;
    return sign | 0x7e00u | (uint16_t)((ax >> 13) & 0x3ffu); /* quiet, keep payload top */
  }
  if (ax >= 0x477ff000u) return sign | 0x7c00u; /* >= 65520 rounds to inf */
  if (ax < 0x33000001u) return sign;            /* <= 2^-25 rounds to zero */
  int e = (int)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7fffffu) | 0x800000u; /* 24-bit significand */
  int shift;                                 /* bits to drop */
  uint32_t base;
  if (e < -14) { /* subnormal result */
    shift = 13 + (-14 - e);
    base = 0;
  } else {
    shift = 13;
    base = (uint32_t)(e + 15) << 10;
    m &= 0x7fffffu;
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  uint32_t r = base + q; /* carry out of the mantissa bumps the exponent: correct */
  if (rem > half || (rem == half && (r & 1u))) r++;
  return sign | (uint16_t)r;
}

float oracle_bf16_to_float(uint16_t b) {
  uint32_t x = (uint32_t)b << 16;
  float f;
  memcpy(&f, &x, 4);
  return f;
}

uint16_t oracle_float_to_bf16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  if ((x & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((x >> 16) | 0x0040u); /* quiet nan */
  uint32_t lsb = (x >> 16) & 1u;
  x += 0x7fffu + lsb;
  return (uint16_t)(x >> 16);
}

/* ------------------------------------------------- binary element loops */
/* The loops mirror flagcx/service/utils.h:681-709: c[i] = a[i] OP b[i] with
 * std::min(a,b) = (b<a)?b:a and std::max(a,b) = (a<b)?b:a.  Integer sum/prod are
 * done on the unsigned type of the same width so that overflow wraps instead of
 * being undefined (same bits as the reference wherever the reference is defined). */

#define LOOP_ARITH(NAME, T, UT, EXPR)                                          \
  static void NAME(void *res, const void *op1, const void *op2, size_t n) {    \
    const T *a = (const T *)op1;                                               \
    const T *b = (const T *)op2;                                               \
    T *c = (T *)res;                                                           \
    for (size_t i = 0; i < n; i++) {                                           \
      UT x = (UT)a[i], y = (UT)b[i];                                           \
      c[i] = (T)(EXPR);                                                        \
    }                                                                          \
  }
#define LOOP_SEL(NAME, T, COND)                                                \
  static void NAME(void *res, const void *op1, const void *op2, size_t n) {    \
    const T *a = (const T *)op1;                                               \
    const T *b = (const T *)op2;                                               \
    T *c = (T *)res;                                                           \
    for (size_t i = 0; i < n; i++) {                                           \
      T x = a[i], y = b[i];                                                    \
      c[i] = (COND) ? y : x;                                                   \
    }                                                                          \
  }
#define ALL_OPS(SFX, T, UT)                                                    \
  LOOP_ARITH(sum_##SFX, T, UT, x + y)                                          \
  LOOP_ARITH(prod_##SFX, T, UT, x * y)                                         \
  LOOP_SEL(min_##SFX, T, y < x)                                                \
  LOOP_SEL(max_##SFX, T, x < y)

ALL_OPS(i8, int8_t, uint8_t)
ALL_OPS(u8, uint8_t, uint8_t)
ALL_OPS(i32, int32_t, uint32_t)
ALL_OPS(u32, uint32_t, uint32_t)
ALL_OPS(i64, int64_t, uint64_t)
ALL_OPS(u64, uint64_t, uint64_t)
ALL_OPS(f32, float, float)
ALL_OPS(f64, double, double)

/* fp16 / bf16 binary: widen, operate in fp32, round once (extension). */
#define HALF_OPS(SFX, TOF, FROMF)                                              \
  static void sum_##SFX(void *res, const void *op1, const void *op2, size_t n) { \
    const uint16_t *a = op1, *b = op2; uint16_t *c = res;                      \
    for (size_t i = 0; i < n; i++) c[i] = FROMF(TOF(a[i]) + TOF(b[i]));        \
  }                                                                            \
  static void prod_##SFX(void *res, const void *op1, const void *op2, size_t n) { \
    const uint16_t *a = op1, *b = op2; uint16_t *c = res;                      \
    for (size_t i = 0; i < n; i++) c[i] = FROMF(TOF(a[i]) * TOF(b[i]));        \
  }                                                                            \
  static void min_##SFX(void *res, const void *op1, const void *op2, size_t n) { \
    const uint16_t *a = op1, *b = op2; uint16_t *c = res;                      \
    for (size_t i = 0; i < n; i++) c[i] = (TOF(b[i]) < TOF(a[i])) ? b[i] : a[i]; \
  }                                                                            \
  static void max_##SFX(void *res, const void *op1, const void *op2, size_t n) { \
    const uint16_t *a = op1, *b = op2; uint16_t *c = res;                      \
    for (size_t i = 0; i < n; i++) c[i] = (TOF(a[i]) < TOF(b[i])) ? b[i] : a[i]; \
  }
HALF_OPS(f16, oracle_half_to_float, oracle_float_to_half)
HALF_OPS(bf16, oracle_bf16_to_float, oracle_float_to_bf16)

typedef void (*binfn)(void *, const void *, const void *, size_t);

static binfn pick(int op, int dtype) {
#define ROW(SFX) { sum_##SFX, prod_##SFX, max_##SFX, min_##SFX }
  static const binfn table[10][4] = {
      ROW(i8), ROW(u8), ROW(i32), ROW(u32), ROW(i64),
      ROW(u64), ROW(f16), ROW(f32), ROW(f64), ROW(bf16)};
#undef ROW
  if (dtype < 0 || dtype > 9 || op < 0 || op > 3) return NULL;
  return table[dtype][op];
}

int oracle_binary(int op, int dtype, void *res, const void *op1, const void *op2,
                  size_t n, int strict) {
  /* op switch of bootstrap.cc:649-671, then dtype switch of utils.h:648-679 */
  if (strict) {
    if (!(op == OP_SUM || op == OP_MAX || op == OP_MIN)) return R_INVALID;
    if (dtype == T_F16 || dtype == T_BF16) return R_INVALID;
  }
  binfn f = pick(op, dtype);
  if (!f) return R_INVALID;
  f(res, op1, op2, n);
  return R_OK;
}

/* ----------------------------------------------------------- N-way fold */

static void fold_half(const void *const *srcs, int k, void *dst, size_t n,
                      int dtype, int op) {
  uint16_t *out = (uint16_t *)dst;
  for (size_t i = 0; i < n; i++) {
    uint16_t b0 = ((const uint16_t *)srcs[0])[i];
    float acc = dtype == T_F16 ? oracle_half_to_float(b0) : oracle_bf16_to_float(b0);
    for (int j = 1; j < k; j++) {
      uint16_t bj = ((const uint16_t *)srcs[j])[i];
      float x = dtype == T_F16 ? oracle_half_to_float(bj) : oracle_bf16_to_float(bj);
      acc = (op == OP_PROD) ? x * acc : x + acc;
    }
    if (op == OP_AVG) acc = acc / (float)k;
    out[i] = dtype == T_F16 ? oracle_float_to_half(acc) : oracle_float_to_bf16(acc);
  }
}

static void divide_by_k(void *dst, size_t n, int dtype, int k) {
  size_t i;
  switch (dtype) {
    case T_I8: { int8_t *p = dst; for (i = 0; i < n; i++) p[i] = (int8_t)(p[i] / k); } break;
    case T_U8: { uint8_t *p = dst; for (i = 0; i < n; i++) p[i] = (uint8_t)(p[i] / (unsigned)k); } break;
    case T_I32: { int32_t *p = dst; for (i = 0; i < n; i++) p[i] = p[i] / k; } break;
    case T_U32: { uint32_t *p = dst; for (i = 0; i < n; i++) p[i] = p[i] / (uint32_t)k; } break;
    case T_I64: { int64_t *p = dst; for (i = 0; i < n; i++) p[i] = p[i] / (int64_t)k; } break;
    case T_U64: { uint64_t *p = dst; for (i = 0; i < n; i++) p[i] = p[i] / (uint64_t)k; } break;
    case T_F32: { float *p = dst; for (i = 0; i < n; i++) p[i] = p[i] / (float)k; } break;
    case T_F64: { double *p = dst; for (i = 0; i < n; i++) p[i] = p[i] / (double)k; } break;
    default: break;
  }
}

int oracle_reduce(const void *const *srcs, int k, void *dst, size_t n, int dtype,
                  int op) {
  size_t ts = oracle_type_size(dtype);
  if (!ts || k < 1 || op < 0 || op > OP_AVG) return R_INVALID;
  int half = (dtype == T_F16 || dtype == T_BF16);
  if (half && (op == OP_SUM || op == OP_PROD || op == OP_AVG)) {
    fold_half(srcs, k, dst, n, dtype, op);
    return R_OK;
  }
  /* (k-1) pairwise passes through an accumulator buffer, op1 = new input,
   * op2 = partial, exactly as the ring loop does (bootstrap.cc:651-653);
   * nranks == 1 is a memcpy (bootstrap.cc:816-821). */
  if (dst != srcs[0]) memmove(dst, srcs[0], n * ts);
  int bop = (op == OP_AVG) ? OP_SUM : op;
  for (int j = 1; j < k; j++) {
    int r = oracle_binary(bop, dtype, dst, srcs[j], dst, n, 0);
    if (r) return r;
  }
  if (op == OP_AVG) divide_by_k(dst, n, dtype, k);
  return R_OK;
}

/* ------------------------------------------------------------ ring code */

void oracle_ring_chunk_table(size_t size, size_t type_size, int nranks,
                             size_t *offset, size_t *length) {
  /* bootstrap.cc:692 MIN_CHUNK_SIZE, :719-722 ChunkBytes, :727-738 table */
  const size_t min_chunk = 1024u * 1024u * 4u;
  size_t chunk = (size + (size_t)nranks - 1) / (size_t)nranks;
  if (chunk < min_chunk) chunk = min_chunk;
  size_t rem = chunk % type_size;
  if (rem) chunk += type_size - rem;
  for (int i = 0; i < nranks; i++) {
    if (chunk * (size_t)i >= size) {
      offset[i] = size;
      length[i] = 0;
      continue;
    }
    offset[i] = chunk * (size_t)i;
    length[i] = chunk * (size_t)(i + 1) >= size ? size - chunk * (size_t)i : chunk;
  }
}

int oracle_ring_reduce_scatter(const void *const *sendbuffs, void *const *recvbuffs,
                               int nranks, const size_t *offset,
                               const size_t *length, int dtype, int op,
                               int strict) {
  size_t ts = oracle_type_size(dtype);
  int half = (dtype == T_F16 || dtype == T_BF16);
  if (nranks < 1 || nranks > 64) return R_INVALID;
  if (strict) {
    /* the first reduce the ring attempts fails on these (utils.h:674-678,
     * bootstrap.cc:668-670); with nranks == 1 the loop body never runs */
    if (nranks > 1 && (!ts || half || !(op == OP_SUM || op == OP_MAX || op == OP_MIN)))
      return R_INVALID;
  } else if (!ts || op < 0 || op > OP_AVG) {
    return R_INVALID;
  }
  if (!strict && (half || op == OP_AVG || op == OP_PROD)) {
    /* extension: evaluate each rank's chunk as one fold in the ring's order */
    for (int rank = 0; rank < nranks; rank++) {
      const void *ord[64];
      for (int j = 0; j < nranks; j++)
        ord[j] = (const char *)sendbuffs[(rank + 1 + j) % nranks] + offset[rank];
      int r = oracle_reduce(ord, nranks, recvbuffs[rank], length[rank] / ts, dtype, op);
      if (r) return r;
    }
    return R_OK;
  }
  size_t sub = 0;
  for (int i = 0; i < nranks; i++) if (length[i] > sub) sub = length[i];
  /* per-rank temp buffers data_for_send / data_for_recv (bootstrap.cc:576-588) */
  char **snd = calloc((size_t)nranks, sizeof(char *));
  char **rcv = calloc((size_t)nranks, sizeof(char *));
  for (int r = 0; r < nranks; r++) {
    snd[r] = calloc(sub ? sub : 1, 1);
    rcv[r] = calloc(sub ? sub : 1, 1);
  }
  int rc = R_OK;
  for (int iter = 0; iter < nranks - 1 && !rc; iter++) {
    /* step 1 for every rank (bootstrap.cc:597-621) */
    for (int rank = 0; rank < nranks; rank++) {
      int send_no = (rank + 2 * nranks - iter - 1) % nranks;
      int recv_no = (rank + 2 * nranks - iter - 2) % nranks;
      int need_send = length[send_no] != 0, need_recv = length[recv_no] != 0;
      if (!need_send && !need_recv) continue;
      if (need_send) {
        if (iter == 0) {
          memcpy(snd[rank], (const char *)sendbuffs[rank] + offset[send_no], length[send_no]);
        } else {
          char *t = snd[rank]; snd[rank] = rcv[rank]; rcv[rank] = t;
        }
      }
    }
    /* step 2: rank sends to next = rank+1, receives from prev (bootstrap.cc:624-637) */
    for (int rank = 0; rank < nranks; rank++) {
      int recv_no = (rank + 2 * nranks - iter - 2) % nranks;
      if (length[recv_no] == 0) continue;
      int prev = (rank + nranks - 1) % nranks;
      memcpy(rcv[rank], snd[prev], length[recv_no]);
    }
    /* step 3: res = OP(local chunk, received partial) into data_for_recv (:648-671) */
    for (int rank = 0; rank < nranks && !rc; rank++) {
      int recv_no = (rank + 2 * nranks - iter - 2) % nranks;
      if (length[recv_no] == 0) continue;
      rc = oracle_binary(op, dtype, rcv[rank],
                         (const char *)sendbuffs[rank] + offset[recv_no], rcv[rank],
                         length[recv_no] / ts, strict);
    }
  }
  if (!rc)
    for (int rank = 0; rank < nranks; rank++) /* bootstrap.cc:677 */
      memcpy(recvbuffs[rank], rcv[rank], length[rank]);
  for (int r = 0; r < nranks; r++) { free(snd[r]); free(rcv[r]); }
  free(snd); free(rcv);
  return rc;
}

int oracle_ring_allreduce(const void *const *sendbuffs, void *recvbuff, int nranks,
                          size_t count, int dtype, int op, int strict) {
  size_t ts = oracle_type_size(dtype);
  if (nranks == 1) { /* bootstrap.cc:816-821: no dtype/op check happens */
    size_t bytes = count * ts;
    if (sendbuffs[0] != recvbuff) memcpy(recvbuff, sendbuffs[0], bytes);
    return R_OK;
  }
  if (!ts) return R_INVALID;
  size_t size = count * ts;
  size_t *offset = calloc((size_t)nranks, sizeof(size_t));
  size_t *length = calloc((size_t)nranks, sizeof(size_t));
  void **outs = calloc((size_t)nranks, sizeof(void *));
  oracle_ring_chunk_table(size, ts, nranks, offset, length);
  /* reduce-scatter writes rank r's chunk at recvbuff + offset[r] (bootstrap.cc:741-743);
   * the all-gather (:746-747) then gives every rank all chunks: one buffer here. */
  char *tmp = malloc(size ? size : 1);
  for (int r = 0; r < nranks; r++) outs[r] = tmp + offset[r];
  int rc = oracle_ring_reduce_scatter(sendbuffs, outs, nranks, offset, length, dtype, op, strict);
  if (!rc) memcpy(recvbuff, tmp, size);
  free(tmp); free(offset); free(length); free(outs);
  return rc;
}

int oracle_reduce_scatter_rank(const void *const *sendbuffs, void *recvbuff,
                               int nranks, int rank, size_t recvcount, int dtype,
                               int op, int strict) {
  size_t ts = oracle_type_size(dtype);
  if (nranks == 1) { /* bootstrap.cc:856-861 */
    if (sendbuffs[0] != recvbuff) memcpy(recvbuff, sendbuffs[0], recvcount * ts);
    return R_OK;
  }
  if (!ts) return R_INVALID;
  size_t bytes = recvcount * ts;
  size_t *offset = calloc((size_t)nranks, sizeof(size_t));
  size_t *length = calloc((size_t)nranks, sizeof(size_t));
  void **outs = calloc((size_t)nranks, sizeof(void *));
  for (int i = 0; i < nranks; i++) { /* bootstrap.cc:862-868 */
    offset[i] = (size_t)i * bytes;
    length[i] = bytes;
    outs[i] = malloc(bytes ? bytes : 1);
  }
  int rc = oracle_ring_reduce_scatter(sendbuffs, outs, nranks, offset, length, dtype, op, strict);
  if (!rc) memcpy(recvbuff, outs[rank], bytes);
  for (int i = 0; i < nranks; i++) free(outs[i]);
  free(offset); free(length); free(outs);
  return rc;
}

/* -------------------------------------------------------- byte movers */

void oracle_refresh(void *buff, size_t start, size_t offset, size_t count,
                    size_t totalcount, size_t ts, int op) {
  /* c2c_algo.cc:590-606: only for sum; two memsets around [offset, offset+count) */
  if (op != OP_SUM) return;
  char *p = (char *)buff + start * ts;
  memset(p, 0, offset * ts);
  memset(p + (offset + count) * ts, 0, (totalcount - offset - count) * ts);
}

void oracle_pack(void *dst, const void *src, size_t nchunks, size_t chunkbytes,
                 size_t srcstride) {
  for (size_t c = 0; c < nchunks; c++)
    memcpy((char *)dst + c * chunkbytes, (const char *)src + c * srcstride, chunkbytes);
}

void oracle_unpack(void *dst, const void *src, size_t nchunks, size_t chunkbytes,
                   size_t dststride) {
  for (size_t c = 0; c < nchunks; c++)
    memcpy((char *)dst + c * dststride, (const char *)src + c * chunkbytes, chunkbytes);
}

/* ------------------------------------------------------- timing helper */

struct job {
  const void *srcs[64];
  void *dst;
  size_t n;
  int k, dtype, op;
};

static void *job_main(void *p) {
  struct job *j = (struct job *)p;
  oracle_reduce(j->srcs, j->k, j->dst, j->n, j->dtype, j->op);
  return NULL;
}

static int cmp_double(const void *a, const void *b) {
  double x = *(const double *)a, y = *(const double *)b;
  return (x > y) - (x < y);
}

double oracle_time_reduce(const void *const *srcs, int k, void *dst, size_t n,
                          int dtype, int op, int nthreads, int warmup, int iters) {
  size_t ts = oracle_type_size(dtype);
  if (!ts || k < 1 || k > 64 || nthreads < 1 || nthreads > 256 || iters < 1) return -1.0;
  struct job *jobs = calloc((size_t)nthreads, sizeof(struct job));
  pthread_t *th = calloc((size_t)nthreads, sizeof(pthread_t));
  double *t = calloc((size_t)iters, sizeof(double));
  size_t per = (n + (size_t)nthreads - 1) / (size_t)nthreads;
  for (int i = 0; i < nthreads; i++) {
    size_t lo = per * (size_t)i, hi = lo + per;
    if (lo > n) lo = n;
    if (hi > n) hi = n;
    for (int j = 0; j < k; j++) jobs[i].srcs[j] = (const char *)srcs[j] + lo * ts;
    jobs[i].dst = (char *)dst + lo * ts;
    jobs[i].n = hi - lo;
    jobs[i].k = k; jobs[i].dtype = dtype; jobs[i].op = op;
  }
  for (int it = -warmup; it < iters; it++) {
    struct timespec a, b;
    clock_gettime(CLOCK_MONOTONIC, &a);
    if (nthreads == 1) {
      job_main(&jobs[0]);
    } else {
      for (int i = 0; i < nthreads; i++) pthread_create(&th[i], NULL, job_main, &jobs[i]);
      for (int i = 0; i < nthreads; i++) pthread_join(th[i], NULL);
    }
    clock_gettime(CLOCK_MONOTONIC, &b);
    if (it >= 0) t[it] = (double)(b.tv_sec - a.tv_sec) + 1e-9 * (double)(b.tv_nsec - a.tv_nsec);
  }
  qsort(t, (size_t)iters, sizeof(double), cmp_double);
  double med = t[iters / 2];
  free(jobs); free(th); free(t);
  return med;
}
