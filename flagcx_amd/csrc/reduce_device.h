// reduce_device.h - gfx950 device code of the N-way elementwise reduction.
//
// One launch folds K input buffers into one output buffer:
//   acc = in[0][i]; for j = 1..K-1: acc = OP(in[j][i], acc); out[i] = finish(acc)
// which is the order and the operand placement (op1 = new input, op2 = partial)
// of the reference's host ring (flagcx/service/bootstrap.cc:651-653) over its
// binary templates (flagcx/service/utils.h:681-709).
//
// Streaming layout: a workgroup is ONE wavefront (64 lanes).  A lane owns one
// 16-byte vector per load, so a wavefront-wide load is one coalesced 1 KiB
// request; the wavefront's tile is U consecutive KiB of every input (U = 1 in the
// shipped configuration), and all K*U loads are issued, input by input, before
// the first use.  Loads carry the `nt` cache hint (streamed once), stores go out
// with `sc1`.  The launch reserves LDS it never touches, only to cap how many
// wavefronts share a CU: with K = 8 inputs 16 resident wavefronts per CU (128 KiB
// of loads in flight) keep HBM busy while staying out of each other's DRAM pages,
// and measured faster than a full CU or a persistent grid; with one or two inputs
// no cap is needed.  No MFMA: (K+1)*16 bytes move per lane per step against a
// handful of VALU ops.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace flagcx_amd {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

enum : int { kSum = 0, kProd = 1, kMax = 2, kMin = 3, kAvg = 4 };
// Internal to the library (no flagcxRedOp_t value): the sum of a member list of which only
// some members are read because the others are known to hold nothing but zeros.  The fold
// over the full list differs from the fold over the members read in one thing only: a sum
// whose addends are all -0.0 comes out +0.0 once a +0.0 takes part, wherever in the list it
// stands.  So the members read are summed in their order and +0.0 is added once at the end,
// before the one rounding of the 16-bit types.  Floating-point types only; an integer
// sum needs nothing of the kind.
enum : int { kSumZ = 5 };

// Element tags for the two 16-bit float formats (raw bit carriers).
struct f16 { uint16_t bits; };
struct bf16 { uint16_t bits; };

#define FLAGCX_MAX_RANKS 64

template <int K>
struct ReduceParams {
  const void *src[K];
  void *dst;
  uint64_t nvec;   // 16-byte vectors in the aligned body
  uint64_t head;   // elements before the body
  uint64_t tail;   // elements after the body
  int32_t k;       // number of inputs actually used (== K except generic)
  int32_t inflight; // 1..3 (< K): a wavefront keeps the loads of at most that many inputs in flight; 0: of all K
  // (32-bit fields: narrower kernel arguments are fetched with vector loads at the start of every wavefront)
  uint32_t lead;   // bytes by which the first tile is shortened, so that every later tile starts on a 128-byte line of dst
  uint32_t run;    // consecutive tiles that stay on one XCD (1: tile = workgroup number)
};

// ------------------------------------------------------------------ widen
__device__ __forceinline__ float widen(f16 h) {
  _Float16 v;
  __builtin_memcpy(&v, &h.bits, 2);
  return (float)v; // v_cvt_f32_f16: exact, subnormals kept
}
__device__ __forceinline__ float widen(bf16 b) {
  return __builtin_bit_cast(float, (uint32_t)b.bits << 16);
}
__device__ __forceinline__ void narrow(float f, f16 &out) {
  _Float16 v = (_Float16)f; // v_cvt_f16_f32: round to nearest even
  __builtin_memcpy(&out.bits, &v, 2);
}
__device__ __forceinline__ void narrow(float f, bf16 &out) {
  uint32_t x = __builtin_bit_cast(uint32_t, f);
  uint32_t r = x + 0x7fffu + ((x >> 16) & 1u); // round to nearest even
  uint32_t q = (x >> 16) | 0x40u;              // quiet NaN keeps sign and top payload
  out.bits = (uint16_t)(((x & 0x7fffffffu) > 0x7f800000u) ? q : (r >> 16));
}

// ---------------------------------------------------------- accumulators
// Acc<T,OP>::type is what the fold carries: fp32 for half-type arithmetic, the
// unsigned twin for integer arithmetic (wraps instead of overflowing), T itself
// for min/max (the selected input is returned bit for bit).
template <typename T> struct Unsigned { typedef T type; };
template <> struct Unsigned<int8_t> { typedef uint8_t type; };
template <> struct Unsigned<int32_t> { typedef uint32_t type; };
template <> struct Unsigned<int64_t> { typedef uint64_t type; };

template <typename T> struct IsHalf { static constexpr bool value = false; };
template <> struct IsHalf<f16> { static constexpr bool value = true; };
template <> struct IsHalf<bf16> { static constexpr bool value = true; };

template <typename T, int OP, bool HALF = IsHalf<T>::value, bool SEL = (OP == kMax || OP == kMin)>
struct Fold;

// min / max on ordinary types
template <typename T, int OP>
struct Fold<T, OP, false, true> {
  typedef T acc_t;
  static __device__ __forceinline__ acc_t init(T x) { return x; }
  static __device__ __forceinline__ acc_t step(T a, acc_t b) {
    // std::max(a,b) = (a<b)?b:a ; std::min(a,b) = (b<a)?b:a
    return (OP == kMax) ? ((a < b) ? b : a) : ((b < a) ? b : a);
  }
  static __device__ __forceinline__ T fin(acc_t acc, int) { return acc; }
};

// min / max on fp16 / bf16: compare widened, keep the chosen bits
template <typename T, int OP>
struct Fold<T, OP, true, true> {
  struct acc_t { T bits; float val; };
  static __device__ __forceinline__ acc_t init(T x) { return {x, widen(x)}; }
  static __device__ __forceinline__ acc_t step(T a, acc_t b) {
    float av = widen(a);
    bool take_b = (OP == kMax) ? (av < b.val) : (b.val < av);
    return take_b ? b : acc_t{a, av};
  }
  static __device__ __forceinline__ T fin(acc_t acc, int) { return acc.bits; }
};

// sum / prod / avg on ordinary types
template <typename T, int OP>
struct Fold<T, OP, false, false> {
  typedef typename Unsigned<T>::type acc_t;
  static __device__ __forceinline__ acc_t init(T x) { return (acc_t)x; }
  static __device__ __forceinline__ acc_t step(T a, acc_t b) {
    return (OP == kProd) ? (acc_t)((acc_t)a * b) : (acc_t)((acc_t)a + b);
  }
  static __device__ __forceinline__ T fin(acc_t acc, int k) {
    if (OP == kSumZ) acc = (acc_t)(acc + (acc_t)0); // -0.0 -> +0.0, every other value unchanged
    return (OP == kAvg) ? (T)((T)acc / (T)k) : (T)acc;
  }
};

// sum / prod / avg on fp16 / bf16: fp32 accumulator, one rounding
template <typename T, int OP>
struct Fold<T, OP, true, false> {
  typedef float acc_t;
  static __device__ __forceinline__ acc_t init(T x) { return widen(x); }
  static __device__ __forceinline__ acc_t step(T a, acc_t b) {
    return (OP == kProd) ? widen(a) * b : widen(a) + b;
  }
  static __device__ __forceinline__ T fin(acc_t acc, int k) {
    if (OP == kAvg) acc = acc / (float)k;
    if (OP == kSumZ) acc = acc + 0.0f;
    T out;
    narrow(acc, out);
    return out;
  }
};

// --------------------------------------------------------- vector plumbing
template <typename T>
union Vec16 {
  u32x4 v;
  T e[16 / sizeof(T)];
};

// 8-bit elements are folded four at a time in a 32-bit word: the bytes at even and
// at odd positions are accumulated apart, as the two 16-bit halves of one word each
// (packed 16-bit instructions; gfx950 has no packed 8-bit ones).  Sums and products
// wrap modulo 256, so whatever gathers above the low byte of a half is dropped when
// the halves are put together again; minima and maxima compare the byte in the HIGH
// position of its half, the other byte cleared, which keeps a signed byte's sign
// where a signed 16-bit compare looks for it.  The results are those of the
// element-by-element fold; written this way the data stays packed, where the
// compiler, left to itself, unpacks eight inputs into one register per byte.
#ifndef FLAGCX_PACKED_8BIT
#define FLAGCX_PACKED_8BIT 1
#endif
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
typedef short i16x2 __attribute__((ext_vector_type(2)));

template <typename T, int OP>
struct Fold8 {
  static_assert(sizeof(T) == 1, "8-bit element types only");
  static constexpr bool kSel = (OP == kMax || OP == kMin);
  static constexpr bool kSigned = ((T)-1 < (T)0);
  struct acc_t { uint32_t ev, od; };
  static __device__ __forceinline__ uint32_t shr8(uint32_t w) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, w) >> (u16x2)(8));
  }
  static __device__ __forceinline__ uint32_t shl8(uint32_t w) {
    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(u16x2, w) << (u16x2)(8));
  }
  static __device__ __forceinline__ uint32_t evenOf(uint32_t w) { return kSel ? (kSigned ? shl8(w) : (w & 0x00ff00ffu)) : w; }
  static __device__ __forceinline__ uint32_t oddOf(uint32_t w) { return kSel ? (w & 0xff00ff00u) : shr8(w); }
  static __device__ __forceinline__ uint32_t join(uint32_t a, uint32_t b) {
    if (kSel) {
      if (kSigned) {
        const i16x2 x = __builtin_bit_cast(i16x2, a), y = __builtin_bit_cast(i16x2, b);
        return __builtin_bit_cast(uint32_t, OP == kMax ? __builtin_elementwise_max(x, y) : __builtin_elementwise_min(x, y));
      }
      const u16x2 x = __builtin_bit_cast(u16x2, a), y = __builtin_bit_cast(u16x2, b);
      return __builtin_bit_cast(uint32_t, OP == kMax ? __builtin_elementwise_max(x, y) : __builtin_elementwise_min(x, y));
    }
    const u16x2 x = __builtin_bit_cast(u16x2, a), y = __builtin_bit_cast(u16x2, b);
    return __builtin_bit_cast(uint32_t, OP == kProd ? (u16x2)(x * y) : (u16x2)(x + y));
  }
  static __device__ __forceinline__ acc_t init(uint32_t w) { return {evenOf(w), oddOf(w)}; }
  static __device__ __forceinline__ acc_t step(uint32_t w, acc_t b) { return {join(evenOf(w), b.ev), join(oddOf(w), b.od)}; }
  // the four folded bytes (a sum not yet divided for the average)
  static __device__ __forceinline__ uint32_t bytes(acc_t a) {
    if (kSel) return (kSigned ? shr8(a.ev) : a.ev) | a.od;
    return (a.ev & 0x00ff00ffu) | shl8(a.od);
  }
};

// a 16-byte vector at any byte address (the hardware's unaligned access mode serves it)
typedef u32x4 u32x4_unaligned __attribute__((aligned(1)));

// Fold one 16-byte vector position across K registers.
template <typename T, int OP, int K>
__device__ __forceinline__ u32x4 foldVec(const u32x4 (&in)[K], int k) {
  typedef Fold<T, OP> F;
  constexpr int N = 16 / sizeof(T);
  Vec16<T> r;
  if constexpr (sizeof(T) == 1 && FLAGCX_PACKED_8BIT) {
    typedef Fold8<T, OP> F8;
#pragma unroll
    for (int d = 0; d < 4; d++) {
      typename F8::acc_t a = F8::init(in[0][d]);
#pragma unroll
      for (int j = 1; j < K; j++) a = F8::step(in[j][d], a);
      r.v[d] = F8::bytes(a);
    }
    if (OP == kAvg) {
#pragma unroll
      for (int e = 0; e < N; e++) r.e[e] = F::fin((typename F::acc_t)r.e[e], k);
    }
    return r.v;
  }
#pragma unroll
  for (int e = 0; e < N; e++) {
    Vec16<T> x;
    x.v = in[0];
    typename F::acc_t acc = F::init(x.e[e]);
#pragma unroll
    for (int j = 1; j < K; j++) {
      x.v = in[j];
      acc = F::step(x.e[e], acc);
    }
    r.e[e] = F::fin(acc, k);
  }
  return r.v;
}

// One element, inputs addressed individually (head and tail elements).
template <typename T, int OP>
__device__ __forceinline__ void foldScalar(const void *const *src, int k, void *dst, uint64_t i) {
  typedef Fold<T, OP> F;
  typename F::acc_t acc = F::init(((const T *)src[0])[i]);
  for (int j = 1; j < k; j++) acc = F::step(((const T *)src[j])[i], acc);
  ((T *)dst)[i] = F::fin(acc, k);
}

// ------------------------------------------------------------------ kernels

// Cache-policy bits of the buffer instructions on gfx950.
enum : int { kAuxSc0 = 1, kAuxNt = 2, kAuxSc1 = 16 };
constexpr int kLoadAux = kAuxNt;
constexpr int kStoreAux = kAuxSc1;
// Raw buffer descriptor word 3 for gfx9-family: 32-bit data format, no swizzle.
constexpr int kRsrcFlags = 0x00020000;
// Accesses that must not be served from a line some cache has held since before the data
// was written (kernels that start before their inputs are complete): re-fetched and
// written through at system scope.
constexpr int kCoherentLoadAux = kAuxSc0 | kAuxSc1 | kAuxNt;
constexpr int kCoherentStoreAux = kAuxSc0 | kAuxSc1;

// One element read / written at system scope (head and tail elements).
template <int BYTES> struct UintOf;
template <> struct UintOf<1> { typedef uint8_t type; };
template <> struct UintOf<2> { typedef uint16_t type; };
template <> struct UintOf<4> { typedef uint32_t type; };
template <> struct UintOf<8> { typedef uint64_t type; };

template <typename T>
__device__ __forceinline__ T coherentLoad(uint64_t base, uint64_t i) {
  typedef typename UintOf<sizeof(T)>::type U;
  const U bits = __hip_atomic_load(reinterpret_cast<const U *>((uintptr_t)base) + i, __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_SYSTEM);
  T out;
  __builtin_memcpy(&out, &bits, sizeof(T));
  return out;
}
template <typename T>
__device__ __forceinline__ void coherentStore(uint64_t base, uint64_t i, T v) {
  typedef typename UintOf<sizeof(T)>::type U;
  U bits;
  __builtin_memcpy(&bits, &v, sizeof(T));
  __hip_atomic_store(reinterpret_cast<U *>((uintptr_t)base) + i, bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
}

// As foldScalar, every access at system scope.
template <typename T, int OP>
__device__ __forceinline__ void foldScalarCoherent(const void *const *src, int k, void *dst, uint64_t i) {
  typedef Fold<T, OP> F;
  typename F::acc_t acc = F::init(coherentLoad<T>((uint64_t)(uintptr_t)src[0], i));
  for (int j = 1; j < k; j++) acc = F::step(coherentLoad<T>((uint64_t)(uintptr_t)src[j], i), acc);
  coherentStore<T>((uint64_t)(uintptr_t)dst, i, F::fin(acc, k));
}


// Aligned body with K known at compile time; one wavefront per workgroup.
// All pointers share the same address modulo 16; p.head elements precede the
// first vector and p.tail follow the last.  Each tile builds buffer descriptors
// that span exactly its own bytes, so the ragged last tile needs no branches:
// out-of-range lanes load zeros and their stores are dropped by the hardware.
// dst may be one of the inputs: a lane reads its positions before it writes
// them, and no other lane touches them.
// TILED: the first tile may be short and tiles may be dealt out in runs per XCD (p.lead,
// p.run); without it tile = workgroup number from the first body byte on, which is what
// line-aligned buffers take (the extra scalar work at the start of every short-lived
// wavefront costs a percent of bandwidth).
// COHERENT: the inputs were completed while this kernel was already on the GPU; loads are
// re-fetched at system scope.
template <typename T, int OP, int K, int U, bool TILED, bool COHERENT = false>
__device__ __forceinline__ void reduceWaveBody(const ReduceParams<K> &p) {
  constexpr int kLoad = COHERENT ? kCoherentLoadAux : kLoadAux;
  constexpr int N = 16 / sizeof(T);
  constexpr uint32_t kTileBytes = 64u * U * 16u;
  const uint64_t bodyBytes = p.nvec * 16;
  const uint32_t lead = TILED ? p.lead : 0;
  const uint64_t ntiles = (bodyBytes + lead + kTileBytes - 1) / kTileBytes;
  const uint64_t headBytes = p.head * sizeof(T);
  const uint32_t voff = threadIdx.x * 16u;
  // Workgroup b runs on XCD b mod 8, every XCD with an L2 of its own.  Where tiles do
  // not start on a cache line of every buffer, neighbouring tiles share lines: runs of
  // p.run consecutive tiles then stay on one XCD, so that a shared line is fetched into,
  // and written back from, one L2.  The grid is a whole number of rounds of 8 runs.
  const uint64_t run = TILED ? p.run : 1;
  const uint64_t round = 8 * run;
  const uint64_t padded = run > 1 ? (ntiles + round - 1) / round * round : ntiles;

  for (uint64_t b = blockIdx.x; b < padded; b += gridDim.x) {
    uint64_t t = b;
    if (TILED && run > 1) {
      const uint64_t bi = b / 8, bx = b % 8;
      t = ((bi / run) * 8 + bx) * run + bi % run;
      if (t >= ntiles) continue;
    }
    const uint64_t off = TILED ? (t ? t * kTileBytes - lead : 0) : t * kTileBytes;
    const uint64_t left = bodyBytes - off;
    const uint32_t cap = TILED ? (t ? kTileBytes : kTileBytes - lead) : kTileBytes;
    const uint32_t span = left < cap ? (uint32_t)left : cap;
    u32x4 in[U][K];
#pragma unroll
    for (int j = 0; j < K; j++) {
      __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          (void *)((const char *)p.src[j] + headBytes + off), 0, span, kRsrcFlags);
#pragma unroll
      for (int u = 0; u < U; u++)
        in[u][j] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff + u * 1024u, 0, kLoad);
      // K loads issued back to back by every resident wavefront reach DRAM as bursts
      // that thrash the row buffers, worst when the K addresses share a channel
      // group (same bank, K rows).  Waiting until at most inflight-1 earlier inputs
      // are outstanding before asking for the next lets other wavefronts' accesses
      // in between, and needs no timing constant (8 inputs 256 MiB apart, buffers
      // not touched by the previous launch: 78 -> 86 % of peak with two in flight).
      // s_waitcnt fields on gfx9: vmcnt [3:0], expcnt [6:4], lgkmcnt [11:8]; 0x0F70
      // leaves the other two counters alone.
      if (K >= 2 && j + 1 < K && p.inflight) {
        if (p.inflight == 2) __builtin_amdgcn_s_waitcnt(0x0F70 | U);
        else if (p.inflight == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | 0);
        else __builtin_amdgcn_s_waitcnt(0x0F70 | (2 * U));
      }
    }
    __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((char *)p.dst + headBytes + off), 0, span, kRsrcFlags);
#pragma unroll
    for (int u = 0; u < U; u++)
      __builtin_amdgcn_raw_buffer_store_b128(foldVec<T, OP, K>(in[u], K), rd, voff + u * 1024u, 0,
                                             kStoreAux);
  }
  // head and tail elements (fewer than 2*N <= 32): last workgroup, one lane each
  if (blockIdx.x == gridDim.x - 1) {
    const uint64_t edge = p.head + p.tail;
    if (threadIdx.x < edge) {
      uint64_t i = threadIdx.x < p.head ? threadIdx.x : p.head + p.nvec * N + (threadIdx.x - p.head);
      if (COHERENT) foldScalarCoherent<T, OP>(p.src, K, p.dst, i);
      else foldScalar<T, OP>(p.src, K, p.dst, i);
    }
  }
}

template <typename T, int OP, int K, int U, bool TILED>
__global__ void __launch_bounds__(64) reduceWaveKernel(ReduceParams<K> p) {
  reduceWaveBody<T, OP, K, U, TILED>(p);
}

// Several independent reductions of the same type, op and K in one launch:
// blockIdx.y picks the segment, blockIdx.x walks its tiles.  Used where a
// collective is cut into chunks that each have their own pointers or fold order
// (ring all-reduce chunks, pipeline chunks, reduce triggers).
#define FLAGCX_BATCH_MAX 32
template <int K>
struct ReduceBatchParams {
  ReduceParams<K> seg[FLAGCX_BATCH_MAX];
};

template <typename T, int OP, int K, int U, bool TILED>
__global__ void __launch_bounds__(64) reduceBatchKernel(ReduceBatchParams<K> bp) {
  reduceWaveBody<T, OP, K, U, TILED>(bp.seg[blockIdx.y]);
}

// More than eight inputs are consumed in order in batches of eight loads; the
// accumulators stay in registers between batches, so the fold and its single final
// rounding are unchanged.  A batch of C inputs is folded as one chain of C steps in
// straight-line code: C is a template argument (the first batch and those in the
// middle are full, the last one goes through a switch on what is left).  With the
// batch length a run-time bound instead, measured on MI355X at 9..16 inputs of
// 128 MiB: 32-bit integer sum / min / max 65-69 % of the HBM peak and 8-bit min / max
// 56-62 %, where the other types ran at 84-88 % and all do now.
//
// What travels from one batch to the next: the accumulators of one 16-byte position.
// Where an accumulator has the size of an element (every type but the two 16-bit
// floating-point ones) they travel packed in four registers, as the inputs do.
template <typename T, int OP, bool PACKED = sizeof(typename Fold<T, OP>::acc_t) == sizeof(T)>
struct Carry;
template <typename T, int OP>
struct Carry<T, OP, true> {
  typedef typename Fold<T, OP>::acc_t acc_t;
  Vec16<T> v;
  __device__ __forceinline__ acc_t get(int e) const { return (acc_t)v.e[e]; }
  __device__ __forceinline__ void set(int e, acc_t a) { v.e[e] = (T)a; }
};
template <typename T, int OP>
struct Carry<T, OP, false> {
  typedef typename Fold<T, OP>::acc_t acc_t;
  acc_t a[16 / sizeof(T)];
  __device__ __forceinline__ acc_t get(int e) const { return a[e]; }
  __device__ __forceinline__ void set(int e, acc_t x) { a[e] = x; }
};

template <typename T, int OP, int C, bool FIRST, int NI>
__device__ __forceinline__ void foldBatch(const u32x4 (&in)[NI], Carry<T, OP> &acc) {
  static_assert(C >= 1 && C <= NI, "a batch folds the first C of the NI vectors");
  typedef Fold<T, OP> F;
  if constexpr (sizeof(T) == 1) {
    typedef Fold8<T, OP> F8;
#pragma unroll
    for (int d = 0; d < 4; d++) {
      typename F8::acc_t a = FIRST ? F8::init(in[0][d]) : F8::step(in[0][d], F8::init(acc.v.v[d]));
#pragma unroll
      for (int b = 1; b < C; b++) a = F8::step(in[b][d], a);
      acc.v.v[d] = F8::bytes(a);
    }
  } else {
    constexpr int N = 16 / sizeof(T);
#pragma unroll
    for (int e = 0; e < N; e++) {
      Vec16<T> x;
      x.v = in[0];
      typename F::acc_t a = FIRST ? F::init(x.e[e]) : F::step(x.e[e], acc.get(e));
#pragma unroll
      for (int b = 1; b < C; b++) {
        x.v = in[b];
        a = F::step(x.e[e], a);
      }
      acc.set(e, a);
    }
  }
}

// One batch of the aligned kernel for more than eight inputs: C loads, then their fold.
// p.inflight as in reduceWaveBody: a wavefront keeps the loads of at most that many inputs
// in flight before it asks for the next (0: the whole batch at once).
template <typename T, int OP, int C, bool FIRST>
__device__ __forceinline__ void anyBatch(const ReduceParams<FLAGCX_MAX_RANKS> &p, int j0, uint64_t byteOff, uint32_t span,
                                         uint32_t voff, Carry<T, OP> &acc) {
  u32x4 in[C];
#pragma unroll
  for (int b = 0; b < C; b++) {
    __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((const char *)p.src[j0 + b] + byteOff), 0, span, kRsrcFlags);
    in[b] = __builtin_amdgcn_raw_buffer_load_b128(rs, voff, 0, kLoadAux);
    if (b + 1 < C && p.inflight) {
      if (p.inflight == 2) __builtin_amdgcn_s_waitcnt(0x0F70 | 1);
      else if (p.inflight == 1) __builtin_amdgcn_s_waitcnt(0x0F70 | 0);
      else __builtin_amdgcn_s_waitcnt(0x0F70 | 3);
    }
  }
  foldBatch<T, OP, C, FIRST>(in, acc);
}

// Aligned body, k from 8 up to FLAGCX_MAX_RANKS, same streaming shape as above: one
// wavefront per workgroup, one KiB of every input per tile.
// (At most 128 registers: sixteen wavefronts per CU, the most its launcher asks for.)
template <typename T, int OP>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4))) reduceWaveAnyKernel(ReduceParams<FLAGCX_MAX_RANKS> p) {
  typedef Fold<T, OP> F;
  constexpr int N = 16 / sizeof(T);
  constexpr int B = 8;
  constexpr uint32_t kTileBytes = 1024u;
  const int k = p.k; // >= B: the launcher sends fewer inputs to the kernels above
  const uint64_t bodyBytes = p.nvec * 16;
  const uint32_t lead = p.lead; // the first tile is short: the others start on a cache line of most buffers
  const uint64_t ntiles = (bodyBytes + lead + kTileBytes - 1) / kTileBytes;
  const uint64_t headBytes = p.head * sizeof(T);
  const uint32_t voff = threadIdx.x * 16u;
  for (uint64_t t = blockIdx.x; t < ntiles; t += gridDim.x) {
    const uint64_t off = t ? t * kTileBytes - lead : 0;
    const uint64_t left = bodyBytes - off;
    const uint32_t cap = t ? kTileBytes : kTileBytes - lead;
    const uint32_t span = left < cap ? (uint32_t)left : cap;
    Carry<T, OP> acc;
    const uint64_t at = headBytes + off;
    anyBatch<T, OP, B, true>(p, 0, at, span, voff, acc);
    int j0 = B;
    for (; j0 + B <= k; j0 += B) anyBatch<T, OP, B, false>(p, j0, at, span, voff, acc);
    switch (k - j0) { // what is left, the same for every wavefront
      case 1: anyBatch<T, OP, 1, false>(p, j0, at, span, voff, acc); break;
      case 2: anyBatch<T, OP, 2, false>(p, j0, at, span, voff, acc); break;
      case 3: anyBatch<T, OP, 3, false>(p, j0, at, span, voff, acc); break;
      case 4: anyBatch<T, OP, 4, false>(p, j0, at, span, voff, acc); break;
      case 5: anyBatch<T, OP, 5, false>(p, j0, at, span, voff, acc); break;
      case 6: anyBatch<T, OP, 6, false>(p, j0, at, span, voff, acc); break;
      case 7: anyBatch<T, OP, 7, false>(p, j0, at, span, voff, acc); break;
      default: break;
    }
    Vec16<T> r;
#pragma unroll
    for (int e = 0; e < N; e++) r.e[e] = F::fin(acc.get(e), k);
    __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((char *)p.dst + headBytes + off), 0, span, kRsrcFlags);
    __builtin_amdgcn_raw_buffer_store_b128(r.v, rd, voff, 0, kStoreAux);
  }
  if (blockIdx.x == gridDim.x - 1) {
    const uint64_t edge = p.head + p.tail;
    if (threadIdx.x < edge) {
      uint64_t i = threadIdx.x < p.head ? threadIdx.x : p.head + p.nvec * N + (threadIdx.x - p.head);
      foldScalar<T, OP>(p.src, k, p.dst, i);
    }
  }
}

// ------------------------------------------------- sources at other offsets
// The same sources read with ALIGNED 16-byte loads and put in place with lane
// shifts.  The output is tiled like the aligned kernel (64 vectors of 16 bytes per
// wavefront and tile, after p.head elements); output vector v of source j needs
// bytes [16 v + d_j, 16 v + d_j + 16) counted from the source's aligned base, i.e.
// the top of aligned granule v and the bottom of granule v + 1, where d_j = the
// source's offset inside a 16-byte line minus the destination's.  Lane i loads
// granule 64 t + i of every source and takes granule 64 t + i + 1 from lane i + 1;
// lane 63 needs the first granule of the NEXT tile, which one more load with a
// one-granule descriptor brings (only lane 0 of it is in range).
// That granule sits in a cache line which the wavefront of the next tile fetches as
// well.  Workgroup b runs on XCD b mod 8, each XCD with an L2 of its own, so with
// tile = workgroup number the line would come from memory twice (128 bytes more per
// KiB and source: 71-78 % of peak where the aligned kernel reaches 83-85 %).  Tiles
// are therefore dealt out in runs of kShiftRun consecutive tiles per XCD: the
// wavefronts of a run start within a few hundred nanoseconds of each other on one
// XCD, and seven of eight look-ahead granules are L2 hits (runs of 4 measured 2-3
// points lower, runs of 12 and 16 the same or lower; a second full load one granule
// further on instead of the lane shift doubles the L2 traffic: 61 %).
// Descriptors are clipped to the granules that hold source bytes, so nothing
// outside a source's own 16-byte lines is ever read.
constexpr int kShiftRun = 8;

template <int K>
struct ShiftParams {
  const void *base[K]; // source address rounded down to 16, at the first body element
  uint32_t shift[K];   // d_j in bytes, 0..15 (a multiple of the element size)
  uint64_t granules[K]; // aligned 16-byte granules of source j that hold body bytes
  const void *src[K];  // original pointers (head and tail elements)
  void *dst;
  uint64_t nvec, head, tail;
  int32_t inflight; // 2: ask for the next source only when at most one earlier source is outstanding
  uint32_t lead;    // bytes by which the first tile is shortened: later tiles start on a 128-byte line of dst
};

// bytes [4 Q + b, 4 Q + b + 16) of the 32 bytes (lo, hi).  Q is a template argument
// and the caller branches on it (it is wave-uniform): with a run-time register index
// the compiler moves the eight words into LDS and indexes them there.
template <int Q>
__device__ __forceinline__ u32x4 funnel16q(const u32x4 lo, const u32x4 hi, uint32_t b) {
  const uint32_t w0 = Q == 0 ? lo[0] : Q == 1 ? lo[1] : Q == 2 ? lo[2] : lo[3];
  const uint32_t w1 = Q == 0 ? lo[1] : Q == 1 ? lo[2] : Q == 2 ? lo[3] : hi[0];
  const uint32_t w2 = Q == 0 ? lo[2] : Q == 1 ? lo[3] : Q == 2 ? hi[0] : hi[1];
  const uint32_t w3 = Q == 0 ? lo[3] : Q == 1 ? hi[0] : Q == 2 ? hi[1] : hi[2];
  const uint32_t w4 = Q == 0 ? hi[0] : Q == 1 ? hi[1] : Q == 2 ? hi[2] : hi[3];
  u32x4 r;
  r[0] = __builtin_amdgcn_alignbyte(w1, w0, b);
  r[1] = __builtin_amdgcn_alignbyte(w2, w1, b);
  r[2] = __builtin_amdgcn_alignbyte(w3, w2, b);
  r[3] = __builtin_amdgcn_alignbyte(w4, w3, b);
  return r;
}
__device__ __forceinline__ u32x4 funnel16(const u32x4 lo, const u32x4 hi, uint32_t q, uint32_t b) {
  switch (q) {
    case 0: return funnel16q<0>(lo, hi, b);
    case 1: return funnel16q<1>(lo, hi, b);
    case 2: return funnel16q<2>(lo, hi, b);
    default: return funnel16q<3>(lo, hi, b);
  }
}

template <typename T, int OP, int K>
__global__ void __launch_bounds__(64) reduceWaveShiftKernel(ShiftParams<K> p) {
  constexpr int N = 16 / sizeof(T);
  const uint32_t lane = threadIdx.x;
  const uint64_t ntiles = (p.nvec * 16 + p.lead + 1023) / 1024;
  const uint64_t headBytes = p.head * sizeof(T);
  // runs of kShiftRun consecutive tiles on one XCD; the grid is a whole number of
  // rounds of 8 runs (a grid smaller than the tiles takes several passes), tiles beyond
  // the last do nothing
  constexpr uint64_t kRound = 8ull * kShiftRun;
  const uint64_t padded = (ntiles + kRound - 1) / kRound * kRound;
  for (uint64_t b = blockIdx.x; b < padded; b += gridDim.x) {
    const uint64_t bi = b / 8, bx = b % 8;
    const uint64_t t = ((bi / kShiftRun) * 8 + bx) * kShiftRun + bi % kShiftRun;
    if (t >= ntiles) continue;
    // the first tile is short, so that the others start on a line of the destination
    const uint64_t off = t ? t * 1024 - p.lead : 0;
    const uint64_t g0 = off / 16;
    u32x4 cur[K], ahead[K];
#pragma unroll
    for (int j = 0; j < K; j++) {
      const uint64_t left = p.granules[j] > g0 ? p.granules[j] - g0 : 0;
      __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
          (void *)((const char *)p.base[j] + g0 * 16), 0, (uint32_t)(left < 64 ? left : 64) * 16u, kRsrcFlags);
      cur[j] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16u, 0, kLoadAux);
      __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
          (void *)((const char *)p.base[j] + g0 * 16 + 1024), 0, left > 64 ? 16u : 0u, kRsrcFlags);
      ahead[j] = __builtin_amdgcn_raw_buffer_load_b128(ra, lane * 16u, 0, kLoadAux);
      if (p.inflight == 2 && j >= 1 && j < K - 1) {
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
        __builtin_amdgcn_s_waitcnt(0x0f70 | 2); // vmcnt(2): this source's two loads only
        __atomic_signal_fence(__ATOMIC_SEQ_CST);
      }
    }
    u32x4 in[K];
#pragma unroll
    for (int j = 0; j < K; j++) {
      u32x4 hi;
#pragma unroll
      for (int d = 0; d < 4; d++) {
        const uint32_t fromNext = __builtin_amdgcn_readfirstlane(ahead[j][d]); // granule 0 of the next tile
        // wave_shl:1 - lane i reads lane i + 1; lane 63 has no source lane and keeps `old`
        hi[d] = (uint32_t)__builtin_amdgcn_update_dpp((int)fromNext, (int)cur[j][d], 0x130, 0xf, 0xf, false);
      }
      in[j] = funnel16(cur[j], hi, p.shift[j] >> 2, p.shift[j] & 3u);
    }
    const uint64_t left = p.nvec * 16 - off;
    const uint32_t cap = t ? 1024u : 1024u - p.lead;
    __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((char *)p.dst + headBytes + off), 0, left < cap ? (uint32_t)left : cap, kRsrcFlags);
    __builtin_amdgcn_raw_buffer_store_b128(foldVec<T, OP, K>(in, K), rd, lane * 16u, 0, kStoreAux);
  }
  // head and tail elements (fewer than 2*N <= 32): last workgroup, one lane each
  if (blockIdx.x == gridDim.x - 1) {
    const uint64_t edge = p.head + p.tail;
    if (threadIdx.x < edge) {
      uint64_t i = threadIdx.x < p.head ? threadIdx.x : p.head + p.nvec * N + (threadIdx.x - p.head);
      foldScalar<T, OP>(p.src, K, p.dst, i);
    }
  }
}

// The same for more than eight sources: batches as in reduceWaveAnyKernel, every
// source loaded aligned and put in place with lane shifts as above.  Batches of four
// sources, not eight: two loads per source, and with eight the kernel needs 117-148
// registers, which leaves room for 12 wavefronts per CU (measured 36-71 % of peak at
// 9..16 sources of 128 MiB), where this one wants 25 or more (70-77 %).
template <typename T, int OP>
__global__ void __launch_bounds__(64) __attribute__((amdgpu_waves_per_eu(4))) reduceWaveShiftAnyKernel(ShiftParams<FLAGCX_MAX_RANKS> p, int k) {
  typedef Fold<T, OP> F;
  constexpr int N = 16 / sizeof(T);
  constexpr int B = 4; // sources per batch: two loads each, and registers enough left for sixteen wavefronts per CU
  const uint32_t lane = threadIdx.x;
  const uint64_t ntiles = (p.nvec * 16 + p.lead + 1023) / 1024;
  const uint64_t headBytes = p.head * sizeof(T);
  constexpr uint64_t kRound = 8ull * kShiftRun;
  const uint64_t padded = (ntiles + kRound - 1) / kRound * kRound;
  for (uint64_t b = blockIdx.x; b < padded; b += gridDim.x) {
    const uint64_t bi = b / 8, bx = b % 8;
    const uint64_t t = ((bi / kShiftRun) * 8 + bx) * kShiftRun + bi % kShiftRun;
    if (t >= ntiles) continue;
    const uint64_t off = t ? t * 1024 - p.lead : 0;
    const uint64_t g0 = off / 16;
    Carry<T, OP> acc;
    for (int j0 = 0; j0 < k; j0 += B) { // k >= B: the first batch is full
      const int c = k - j0 < B ? k - j0 : B;
      u32x4 cur[B], ahead[B];
#pragma unroll
      for (int i = 0; i < B; i++)
        if (i < c) {
          const int j = j0 + i;
          const uint64_t left = p.granules[j] > g0 ? p.granules[j] - g0 : 0;
          __amdgpu_buffer_rsrc_t rs = __builtin_amdgcn_make_buffer_rsrc(
              (void *)((const char *)p.base[j] + g0 * 16), 0, (uint32_t)(left < 64 ? left : 64) * 16u, kRsrcFlags);
          cur[i] = __builtin_amdgcn_raw_buffer_load_b128(rs, lane * 16u, 0, kLoadAux);
          __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(
              (void *)((const char *)p.base[j] + g0 * 16 + 1024), 0, left > 64 ? 16u : 0u, kRsrcFlags);
          ahead[i] = __builtin_amdgcn_raw_buffer_load_b128(ra, lane * 16u, 0, kLoadAux);
        }
      u32x4 in[B];
#pragma unroll
      for (int i = 0; i < B; i++)
        if (i < c) {
          u32x4 hi;
#pragma unroll
          for (int d = 0; d < 4; d++) {
            const uint32_t fromNext = __builtin_amdgcn_readfirstlane(ahead[i][d]);
            hi[d] = (uint32_t)__builtin_amdgcn_update_dpp((int)fromNext, (int)cur[i][d], 0x130, 0xf, 0xf, false);
          }
          const uint32_t sh = p.shift[j0 + i];
          in[i] = funnel16(cur[i], hi, sh >> 2, sh & 3u);
        }
      if (j0 == 0) foldBatch<T, OP, B, true>(in, acc);
      else if (c == B) foldBatch<T, OP, B, false>(in, acc);
      else if (c == 3) foldBatch<T, OP, 3, false>(in, acc);
      else if (c == 2) foldBatch<T, OP, 2, false>(in, acc);
      else foldBatch<T, OP, 1, false>(in, acc);
    }
    Vec16<T> r;
#pragma unroll
    for (int e = 0; e < N; e++) r.e[e] = F::fin(acc.get(e), k);
    const uint64_t left = p.nvec * 16 - off;
    const uint32_t cap = t ? 1024u : 1024u - p.lead;
    __amdgpu_buffer_rsrc_t rd = __builtin_amdgcn_make_buffer_rsrc(
        (void *)((char *)p.dst + headBytes + off), 0, left < cap ? (uint32_t)left : cap, kRsrcFlags);
    __builtin_amdgcn_raw_buffer_store_b128(r.v, rd, lane * 16u, 0, kStoreAux);
  }
  if (blockIdx.x == gridDim.x - 1) {
    const uint64_t edge = p.head + p.tail;
    if (threadIdx.x < edge) {
      uint64_t i = threadIdx.x < p.head ? threadIdx.x : p.head + p.nvec * N + (threadIdx.x - p.head);
      foldScalar<T, OP>(p.src, k, p.dst, i);
    }
  }
}

} // namespace flagcx_amd
