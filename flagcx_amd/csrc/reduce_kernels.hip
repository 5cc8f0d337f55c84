// reduce_kernels.hip - instantiates the N-way reduce kernels for ONE element type
// and provides its launcher.  Compiled once per type with -DFLAGCX_DT=<enum value>
// so the ten types build in parallel.
#include "launch.h"
#include <hip/hip_ext.h>
#include "reduce_device.h"
#include "reduce_queue_device.h"
#include "reduce_gate_device.h"

#ifndef FLAGCX_DT
#error "compile with -DFLAGCX_DT=<flagcxDataType_t value>"
#endif

namespace flagcx_amd {

#if FLAGCX_DT == 0
typedef int8_t elem_t;
#elif FLAGCX_DT == 1
typedef uint8_t elem_t;
#elif FLAGCX_DT == 2
typedef int32_t elem_t;
#elif FLAGCX_DT == 3
typedef uint32_t elem_t;
#elif FLAGCX_DT == 4
typedef int64_t elem_t;
#elif FLAGCX_DT == 5
typedef uint64_t elem_t;
#elif FLAGCX_DT == 6
typedef f16 elem_t;
#elif FLAGCX_DT == 7
typedef float elem_t;
#elif FLAGCX_DT == 8
typedef double elem_t;
#elif FLAGCX_DT == 9
typedef bf16 elem_t;
#else
#error "unknown FLAGCX_DT"
#endif

#define FLAGCX_CAT2(a, b) a##b
#define FLAGCX_CAT(a, b) FLAGCX_CAT2(a, b)

// Unroll (KiB of each input per wavefront).  One KiB per input measured best or
// equal for every K on MI355X once buffers are large enough to stream from HBM,
// and is the least sensitive to how the inputs' addresses alias in the HBM
// channel hash (tried: inter-buffer strides of 128 MiB .. 1 GiB plus 0 .. 33 MiB).
constexpr int unrollFor(int) { return 1; }

constexpr uint64_t kMaxGrid = 1u << 24;

struct Split {
  uint64_t head, nvec, tail;
  bool vector; // every pointer shares the destination's offset inside a 16-byte line
};

// The body is tiled on the destination: head elements up to its next 16-byte
// line, then whole vectors, then a tail.  Sources at another offset modulo 16
// take the unaligned-load kernel.
static Split splitFor(const ReduceCall &c) {
  constexpr uint64_t N = 16 / sizeof(elem_t);
  Split s{0, 0, 0, true};
  const uintptr_t mis = (uintptr_t)c.dst & 15u;
  for (int j = 0; j < c.k; j++)
    if (((uintptr_t)c.src[j] & 15u) != mis) s.vector = false;
  uint64_t head = ((16u - mis) & 15u) / sizeof(elem_t);
  if (head > c.count) head = c.count;
  s.head = head;
  s.nvec = (c.count - head) / N;
  s.tail = c.count - head - s.nvec * N;
  return s;
}

// Where the tiles start.  All pointers agree modulo 16 here, but not necessarily modulo
// the 128-byte cache line, and a KiB tile that does not start on a line shares its first
// and last line with its neighbours, which run on other XCDs: such a stream costs an
// extra line fetch (or a partial line write) per KiB.  The first tile is cut short by
// `lead` bytes so that all later tiles start on a line of the streams that it pays most
// to have there.  What a stream that straddles costs, fitted to measurements (256 MiB bf16
// per input, percent of peak, tiles on the sources' lines / on the destination's, sources
// 16 bytes into their lines and the destination on one: 2 inputs 77.5 / 83.2, 3: 77.5 /
// 81.5, 4: 78.9 / 82.9, 5: 76.7 / 80.7, 6: 78.2 / 79.2, 7: 78.1 / 79.1, 8: 77.1 / 76.4;
// at 64 MiB per input 6 and 8 inputs: 82-83 / 77): a straddling load stream 1, a
// straddling store stream 5.5 - unless it straddles by exactly half a line (sources 80
// and destination 16 bytes in: 83-85 on the sources' lines for every input count, 80-83
// on the destination's), where whole 64-byte halves are still written: 0.5.  So up to
// five sources follow the destination and six or more outvote it.  Under 96 MiB per input
// it is the other way round (64 MiB, 3 / 5 inputs: 83-84 on the sources' lines, 80-81 on
// the destination's; 128 MiB: 78 / 78-79 against 80 / 80-81) and the destination counts
// as two sources, so two or more sources that agree outvote it.  Every buffer 16 or 64
// bytes into a line: 68 / 74-77 without the short first tile, 83-85 with it (as with
// line-aligned buffers).
// Sources that still straddle get runs of kLineRun consecutive tiles per XCD, so that a
// shared line is fetched into one L2 once (+1 to +3 points; with only the destination
// straddling the runs cost 2 to 6 points and are not used, as they cost 4 with every
// stream on a line).
constexpr uint32_t kLineRun = 8;
template <int K>
static void setTiling(ReduceParams<K> &p, const ReduceCall &c, const Split &s) {
  const uintptr_t headBytes = s.head * sizeof(elem_t);
  uint32_t off[K + 1];
  for (int j = 0; j < K; j++) off[j] = (uint32_t)(((uintptr_t)c.src[j] + headBytes) & 127u);
  off[K] = (uint32_t)(((uintptr_t)c.dst + headBytes) & 127u);
  uint32_t best = off[K];
  int bestCost = 1 << 30;
  // launches of under 96 MiB per input run few rounds of wavefronts and do better on the sources'
  // lines: there the destination counts as two sources
  const int storeCost = s.nvec >= (96ull << 20) / 16 ? 11 : 4;
  for (int i = K; i >= 0; i--) { // the destination's own offset first: it wins ties
    int cost = 0; // in halves of a straddling load stream
    for (int j = 0; j < K; j++) cost += off[j] != off[i] ? 2 : 0;
    const uint32_t apart = (off[K] - off[i]) & 127u;
    cost += apart == 0 ? 0 : apart == 64 && storeCost > 4 ? 1 : storeCost;
    if (cost < bestCost) {
      bestCost = cost;
      best = off[i];
    }
  }
  p.lead = s.nvec ? best : 0; // tile 1 starts 1024 - best bytes in: on a line of the streams that sit `best` bytes into theirs
  bool sourceStraddles = false;
  for (int j = 0; j < K; j++) sourceStraddles = sourceStraddles || off[j] != best;
  p.run = sourceStraddles ? kLineRun : 1;
}

template <int OP, int K>
static int launchFixed(const ReduceCall &c, const Split &s) {
  constexpr int U = unrollFor(K);
  ReduceParams<K> p;
  for (int j = 0; j < K; j++) p.src[j] = c.src[j];
  p.dst = c.dst;
  p.nvec = s.nvec;
  p.head = s.head;
  p.tail = s.tail;
  p.k = K;
  const uint64_t tileBytes = 64ull * U * 16ull;
  // Small messages: a launch of no more workgroups than there are CUs is over in one round of
  // wavefronts, whatever its shape, and what it costs is the host's time per launch (the GPU
  // takes such launches back to back as fast as empty ones).  So no tiling arithmetic, no shape
  // lookup, no LDS reservation (nothing to cap), and one runtime call whose return value is the
  // launch's status.
  if (!c.anyOrder && (s.nvec * 16 + tileBytes - 1) / tileBytes <= (uint64_t)deviceInfo().numCU) {
    p.inflight = 0;
    p.lead = 0;
    p.run = 1;
    uint64_t few = (s.nvec * 16 + tileBytes - 1) / tileBytes;
    if (few < 1) few = 1;
    void *args[] = {&p};
    return (int)hipLaunchKernel(reinterpret_cast<const void *>(&reduceWaveKernel<elem_t, OP, K, U, false>), dim3((unsigned)few),
                                dim3(64), args, 0, c.stream);
  }
  setTiling(p, c, s);
  uint64_t tiles = (s.nvec * 16 + p.lead + tileBytes - 1) / tileBytes;
  // a limit on the inputs in flight per wavefront trades latency per wavefront for
  // DRAM efficiency: by default only where the launch runs many rounds of resident
  // wavefronts
  LaunchShape shape = launchShapeFor(K, tiles);
  // Buffers at different places inside their cache lines (tiles dealt out in runs per XCD):
  // from 48 MiB per input on, two, four and five inputs do better with all loads at once, six
  // and seven with one in flight and more wavefronts.  Measured on MI355X, every source at a
  // place of its own, fp32 / bf16 at 128 MiB per input, percent of peak, shape of the aligned
  // case -> this one: 2 inputs 84 / 78 -> 83 / 80, 4: 79 / 76 -> 86 / 86, 5: 78 / 75 -> 82 / 82,
  // 6: 79 / 76 -> 81 / 76, 7: 77 / 73 -> 79 / 75 (384 MiB: +1 to +5 on the same rows); medians
  // over random places, sizes and types: 82.0 -> 82.8, 80.6 -> 82.8, 77.7 -> 80.3, 80.2 ->
  // 80.9, 78.9 -> 79.8.  Three inputs lost a point that way and eight gained nothing: both keep
  // their shape, and so does a reduce whose output is one of its inputs (five inputs in place:
  // 69 -> 61 %).  Explicit flagcxLocalTune* settings win.
  bool inPlace = false;
  for (int j = 0; j < K; j++) inPlace = inPlace || c.src[j] == c.dst;
  if (p.run > 1 && tiles >= 48 * 1024 && K >= 2 && K <= 7 && K != 3 && !inPlace && tunedWavesPerCU(K) < 0 &&
      tunedLoadsInFlight(K) < 0) {
    shape.loads = K <= 5 ? 0 : 1;
    shape.waves = K == 2 ? 25 : K <= 5 ? 18 : 25;
  }
  p.inflight = shape.loads;
  if (tiles < 1) tiles = 1;
  if (p.run > 1) tiles = (tiles + 8ull * p.run - 1) / (8ull * p.run) * (8ull * p.run);
  if (tiles > kMaxGrid) tiles = kMaxGrid;
  const int lds = ldsReservation(shape.waves);
  if (c.anyOrder) {
    if (p.lead == 0 && p.run == 1)
      hipExtLaunchKernelGGL((reduceWaveKernel<elem_t, OP, K, U, false>), dim3((unsigned)tiles), dim3(64), lds, c.stream,
                            nullptr, nullptr, hipExtAnyOrderLaunch, p);
    else
      hipExtLaunchKernelGGL((reduceWaveKernel<elem_t, OP, K, U, true>), dim3((unsigned)tiles), dim3(64), lds, c.stream,
                            nullptr, nullptr, hipExtAnyOrderLaunch, p);
  } else if (p.lead == 0 && p.run == 1) {
    reduceWaveKernel<elem_t, OP, K, U, false><<<dim3((unsigned)tiles), dim3(64), lds, c.stream>>>(p);
  } else {
    reduceWaveKernel<elem_t, OP, K, U, true><<<dim3((unsigned)tiles), dim3(64), lds, c.stream>>>(p);
  }
  return (int)hipGetLastError();
}

template <int OP>
static int launchAny(const ReduceCall &c, const Split &s) {
  if (c.k <= 8 || c.k > FLAGCX_MAX_RANKS) return (int)hipErrorInvalidValue; // the kernels fold a full first batch of eight
  ReduceParams<FLAGCX_MAX_RANKS> p;
  for (int j = 0; j < c.k; j++) p.src[j] = c.src[j];
  for (int j = c.k; j < FLAGCX_MAX_RANKS; j++) p.src[j] = nullptr;
  p.dst = c.dst;
  p.nvec = s.nvec;
  p.head = s.head;
  p.tail = s.tail;
  p.k = c.k;
  p.inflight = tunedLoadsInFlight(8) >= 0 ? tunedLoadsInFlight(8) : 2;
  p.lead = 0;
  p.run = 1;
  if (s.vector && s.nvec) {
    // the position inside a 128-byte line that most buffers share (the destination counts double)
    const uintptr_t headBytes = s.head * sizeof(elem_t);
    int count[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int j = 0; j < c.k; j++) count[(((uintptr_t)c.src[j] + headBytes) & 127u) >> 4]++;
    count[(((uintptr_t)c.dst + headBytes) & 127u) >> 4] += 2;
    int best = 0;
    for (int i = 1; i < 8; i++)
      if (count[i] > count[best]) best = i;
    p.lead = (uint32_t)best * 16u;
  }
  uint64_t tiles = (s.nvec * 16 + p.lead + 1023) / 1024;
  if (tiles < 1) tiles = 1;
  if (tiles > kMaxGrid) tiles = kMaxGrid;
  // More than eight inputs are loaded eight at a time, each batch paced like the kernels
  // for up to eight: the next input is asked for when at most one earlier one is
  // outstanding, 16 wavefronts per CU up to 160 MiB per input and 14 above.  Measured on
  // MI355X, fp32 and bf16, 9 / 12 / 16 / 32 inputs, percent of peak: 128 MiB per input
  // 85 / 85 / 84 / 83, 256 MiB 85 / 83 / 81 / 80, 512 MiB 82 / 80 / 82 / 80; all eight
  // loads at once with 12 / 10 / 8 wavefronts (the best caps for that) gave 86 / 84 / 84 /
  // 82, 80 / 79 / 77 / 76 and 80 / 79 / 75 / 77.  flagcxLocalTune(8, n) and
  // flagcxLocalTuneLoads(8, n) override.
  const int tuned = tunedWavesPerCU(8);
  const int waves = tuned >= 0 ? tuned : tiles > 160 * 1024 ? 14 : 16;
  if (s.vector) {
    reduceWaveAnyKernel<elem_t, OP><<<dim3((unsigned)tiles), dim3(64), ldsReservation(waves), c.stream>>>(p);
    return (int)hipGetLastError();
  }
  // More than eight sources at another offset modulo 16 than the output (up to eight
  // take reduceWaveShiftKernel): aligned loads and lane shifts, four sources at a time.
  // The kernel wants every wavefront its registers allow (no cap: 12 per CU gave
  // 53-59 % of peak, 16 62-71 %, 25 and more 70-77 %, at 9..32 sources of 128 MiB).
  // Unaligned 16-byte loads instead, measured beside it: 55-61 % on 1- and 2-byte
  // elements at offsets that are no multiple of four, 70-73 % on 4- and 8-byte
  // elements at 128 MiB, 66-70 % at 500 MiB and 56-59 % there when the output is one of
  // the sources, where the lane shifts hold 71-79 %.
  {
    ShiftParams<FLAGCX_MAX_RANKS> q;
    const uint64_t headBytes = s.head * sizeof(elem_t);
    for (int j = 0; j < FLAGCX_MAX_RANKS; j++) {
      const uintptr_t first = j < c.k ? (uintptr_t)c.src[j] + headBytes : 0;
      q.base[j] = (const void *)(first & ~(uintptr_t)15);
      q.shift[j] = (uint32_t)(first & 15u);
      q.granules[j] = j < c.k ? s.nvec + (q.shift[j] ? 1 : 0) : 0;
      q.src[j] = j < c.k ? c.src[j] : nullptr;
    }
    q.dst = c.dst;
    q.nvec = s.nvec;
    q.head = s.head;
    q.tail = s.tail;
    q.inflight = 0;
    q.lead = s.nvec ? (uint32_t)(((uintptr_t)c.dst + headBytes) & 127u) : 0;
    const uint64_t shiftTiles = (s.nvec * 16 + q.lead + 1023) / 1024;
    constexpr uint64_t span = 8ull * kShiftRun;
    uint64_t grid = (shiftTiles + span - 1) / span * span;
    if (grid < span) grid = span;
    if (grid > kMaxGrid) grid = kMaxGrid;
    reduceWaveShiftAnyKernel<elem_t, OP><<<dim3((unsigned)grid), dim3(64), ldsReservation(tuned >= 0 ? tuned : 0), c.stream>>>(q, c.k);
  }
  return (int)hipGetLastError();
}

// Sources at another offset modulo 16 than the output, up to eight of them: aligned
// loads put in place with lane shifts.
template <int OP, int K>
static int launchShift(const ReduceCall &c, const Split &s) {
  ShiftParams<K> p;
  const uint64_t headBytes = s.head * sizeof(elem_t);
  for (int j = 0; j < K; j++) {
    const uintptr_t first = (uintptr_t)c.src[j] + headBytes;
    p.base[j] = (const void *)(first & ~(uintptr_t)15);
    p.shift[j] = (uint32_t)(first & 15u);
    p.granules[j] = s.nvec + (p.shift[j] ? 1 : 0);
    p.src[j] = c.src[j];
  }
  p.dst = c.dst;
  p.nvec = s.nvec;
  p.head = s.head;
  p.tail = s.tail;
  // the first tile is cut short so that the others start on a 128-byte line of the destination
  p.lead = s.nvec ? (uint32_t)(((uintptr_t)c.dst + headBytes) & 127u) : 0;
  const uint64_t tiles = (s.nvec * 16 + p.lead + 1023) / 1024;
  // One tile per wavefront, dealt out in runs of kShiftRun tiles per XCD (whole rounds of
  // 8 runs).  Measured on MI355X, bf16 over rotating buffers, percent of peak at 32 /
  // 128 / 512 MiB per input: 1 input (a misaligned copy) 66 / 77 / 81, 2: 71 / 80 / 83,
  // 3: 70-75 / 80-82 / 83-84, 4: 74-76 / 81 / 84, 6: 75 / 80-82 / 81, 8: 74-76 / 79 / 77-78
  // (tile = workgroup number, two tiles per wavefront: 62-65 / 73-76 / 69-80).
  // Wavefronts per CU: no cap / 25 / 21 / 18 / 14 for up to 2 / 3 / 4 / 5 / 6 inputs (5 inputs at 18 instead of 14:
  // 72 / 80 / 79 -> 75 / 80 / 83); 7 and 8
  // keep two sources in flight per wavefront at 16, which holds 77-79 % from 128 MiB to
  // 1 GiB where all at once falls to 70-73 %.
  constexpr uint64_t span = 8ull * kShiftRun;
  uint64_t grid = (tiles + span - 1) / span * span;
  if (grid < span) grid = span;
  if (grid > kMaxGrid) grid = kMaxGrid; // a multiple of the round: the kernel takes several passes
  const int loads = tunedLoadsInFlight(K);
  p.inflight = loads >= 0 ? (loads == 2 ? 2 : 0) : K >= 7 ? 2 : 0;
  const int tuned = tunedWavesPerCU(K);
  const int lds = ldsReservation(tuned >= 0 ? tuned : K <= 2 ? 0 : K == 3 ? 25 : K == 4 ? 21 : K == 5 ? 18 : K == 6 ? 14 : 16);
  reduceWaveShiftKernel<elem_t, OP, K><<<dim3((unsigned)grid), dim3(64), lds, c.stream>>>(p);
  return (int)hipGetLastError();
}

template <int OP>
static int launchOp(const ReduceCall &c) {
  const Split s = splitFor(c);
  if (!s.vector && c.k <= 8) {
    switch (c.k) {
      case 1: return launchShift<OP, 1>(c, s);
      case 2: return launchShift<OP, 2>(c, s);
      case 3: return launchShift<OP, 3>(c, s);
      case 4: return launchShift<OP, 4>(c, s);
      case 5: return launchShift<OP, 5>(c, s);
      case 6: return launchShift<OP, 6>(c, s);
      case 7: return launchShift<OP, 7>(c, s);
      default: return launchShift<OP, 8>(c, s);
    }
  }
  if (!s.vector || c.k > 8) return launchAny<OP>(c, s);
  switch (c.k) {
    case 1: return launchFixed<OP, 1>(c, s);
    case 2: return launchFixed<OP, 2>(c, s);
    case 3: return launchFixed<OP, 3>(c, s);
    case 4: return launchFixed<OP, 4>(c, s);
    case 5: return launchFixed<OP, 5>(c, s);
    case 6: return launchFixed<OP, 6>(c, s);
    case 7: return launchFixed<OP, 7>(c, s);
    default: return launchFixed<OP, 8>(c, s);
  }
}

template <int OP, int K>
static int launchBatchFixed(const ReduceCall *calls, const Split *splits, int n) {
  constexpr int U = unrollFor(K);
  const uint64_t tileBytes = 64ull * U * 16ull;
  for (int base = 0; base < n; base += FLAGCX_BATCH_MAX) {
    const int m = n - base < FLAGCX_BATCH_MAX ? n - base : FLAGCX_BATCH_MAX;
    ReduceBatchParams<K> bp;
    uint64_t maxTiles = 1, totalTiles = 0;
    for (int i = 0; i < m; i++) {
      const ReduceCall &c = calls[base + i];
      const Split &s = splits[base + i];
      ReduceParams<K> &p = bp.seg[i];
      for (int j = 0; j < K; j++) p.src[j] = c.src[j];
      p.dst = c.dst;
      p.nvec = s.nvec;
      p.head = s.head;
      p.tail = s.tail;
      p.k = K;
      p.inflight = 0;
      setTiling(p, c, s);
      uint64_t tiles = (s.nvec * 16 + p.lead + tileBytes - 1) / tileBytes;
      if (p.run > 1) tiles = (tiles + 8ull * p.run - 1) / (8ull * p.run) * (8ull * p.run);
      if (tiles > maxTiles) maxTiles = tiles;
      totalTiles += tiles;
    }
    if (maxTiles > kMaxGrid) maxTiles = kMaxGrid;
    const LaunchShape shape = launchShapeFor(K, totalTiles);
    for (int i = 0; i < m; i++) bp.seg[i].inflight = shape.loads;
    const int lds = ldsReservation(shape.waves);
    bool tiled = false;
    for (int i = 0; i < m; i++) tiled = tiled || bp.seg[i].lead != 0 || bp.seg[i].run != 1;
    if (tiled)
      reduceBatchKernel<elem_t, OP, K, U, true>
          <<<dim3((unsigned)maxTiles, (unsigned)m), dim3(64), lds, calls[0].stream>>>(bp);
    else
      reduceBatchKernel<elem_t, OP, K, U, false>
          <<<dim3((unsigned)maxTiles, (unsigned)m), dim3(64), lds, calls[0].stream>>>(bp);
    const int err = (int)hipGetLastError();
    if (err) return err;
  }
  return 0;
}

template <int OP>
static int launchBatchOp(const ReduceCall *calls, int n) {
  // One launch per 32 segments when every segment can take the 16-byte path with
  // the same compile-time K; otherwise segment by segment.
  const int k = calls[0].k;
  bool fast = k <= 8 && n > 1;
  Split splits[256];
  if (n > 256) fast = false;
  for (int i = 0; fast && i < n; i++) {
    splits[i] = splitFor(calls[i]);
    if (!splits[i].vector || calls[i].k != k) fast = false;
  }
  if (!fast) {
    for (int i = 0; i < n; i++) {
      const int err = launchOp<OP>(calls[i]);
      if (err) return err;
    }
    return 0;
  }
  switch (k) {
    case 1: return launchBatchFixed<OP, 1>(calls, splits, n);
    case 2: return launchBatchFixed<OP, 2>(calls, splits, n);
    case 3: return launchBatchFixed<OP, 3>(calls, splits, n);
    case 4: return launchBatchFixed<OP, 4>(calls, splits, n);
    case 5: return launchBatchFixed<OP, 5>(calls, splits, n);
    case 6: return launchBatchFixed<OP, 6>(calls, splits, n);
    case 7: return launchBatchFixed<OP, 7>(calls, splits, n);
    default: return launchBatchFixed<OP, 8>(calls, splits, n);
  }
}

// A batch whose workgroups wait for the host's word that their descriptor's inputs are
// complete: one launch, the first tile's workgroup leads.
template <int OP, int K>
static int launchGatedFixed(const ReduceCall *calls, const Split *splits, int n, const GateArgs &g) {
  constexpr int U = unrollFor(K);
  const uint64_t tileBytes = 64ull * U * 16ull;
  ReduceBatchParams<K> bp;
  uint64_t maxTiles = 1, totalTiles = 0;
  for (int i = 0; i < n; i++) {
    const ReduceCall &c = calls[i];
    const Split &s = splits[i];
    ReduceParams<K> &p = bp.seg[i];
    for (int j = 0; j < K; j++) p.src[j] = c.src[j];
    p.dst = c.dst;
    p.nvec = s.nvec;
    p.head = s.head;
    p.tail = s.tail;
    p.k = K;
    setTiling(p, c, s);
    uint64_t tiles = (s.nvec * 16 + p.lead + tileBytes - 1) / tileBytes;
    if (p.run > 1) tiles = (tiles + 8ull * p.run - 1) / (8ull * p.run) * (8ull * p.run);
    if (tiles > maxTiles) maxTiles = tiles;
    totalTiles += tiles;
  }
  if (maxTiles > kMaxGrid) maxTiles = kMaxGrid;
  // Every wavefront reads the gate's count before its loads and holds its slot without
  // traffic meanwhile: somewhat more resident wavefronts than the plain batch launch make
  // up for part of it.  Measured, 128 chunks of 4 MiB per input, TB/s: vector read with the
  // plain batch's shape -> vector read with its own shape -> scalar read with its own shape
  // (the plain batch itself): 2 inputs 5.63 -> 6.13 -> 6.19 (6.53), 3: 5.39 -> 6.26 -> 6.33
  // (6.43), 4: 5.63 -> 6.33 -> 6.45 (6.65), 6: 5.84 -> 6.22 -> 6.44 (6.68), 8: 6.10 -> 6.35
  // -> 6.47 (6.69); shards of 32 chunks gain more from the scalar read (2 inputs 5.9 -> 6.4).
  LaunchShape shape = launchShapeFor(K, totalTiles);
  if (K <= 3) shape.loads = 0;
  if (tunedWavesPerCU(K) < 0)
    shape.waves = g.scalarRead ? (K == 1 ? 0 : K == 2 ? 25 : K == 3 ? 21 : K <= 5 ? 18 : 16)
                               : (K <= 3 ? 0 : K <= 5 ? 21 : 18);
  for (int i = 0; i < n; i++) bp.seg[i].inflight = shape.loads;
  for (int i = n; i < FLAGCX_BATCH_MAX; i++) bp.seg[i] = bp.seg[0];
  const int lds = ldsReservation(shape.waves);
  reduceGatedBatchKernel<elem_t, OP, K, U><<<dim3((unsigned)maxTiles, (unsigned)n), dim3(64), lds, calls[0].stream>>>(bp, g);
  return (int)hipGetLastError();
}

template <int OP>
static int launchGatedOp(const ReduceCall *calls, int n, const GateArgs &g) {
  const int k = calls[0].k;
  if (k > 8 || n < 1 || n > kGateBatchMax) return (int)hipErrorInvalidValue;
  Split splits[kGateBatchMax];
  for (int i = 0; i < n; i++) {
    splits[i] = splitFor(calls[i]);
    if (!splits[i].vector || calls[i].k != k) return (int)hipErrorInvalidValue;
  }
  switch (k) {
    case 1: return launchGatedFixed<OP, 1>(calls, splits, n, g);
    case 2: return launchGatedFixed<OP, 2>(calls, splits, n, g);
    case 3: return launchGatedFixed<OP, 3>(calls, splits, n, g);
    case 4: return launchGatedFixed<OP, 4>(calls, splits, n, g);
    case 5: return launchGatedFixed<OP, 5>(calls, splits, n, g);
    case 6: return launchGatedFixed<OP, 6>(calls, splits, n, g);
    case 7: return launchGatedFixed<OP, 7>(calls, splits, n, g);
    default: return launchGatedFixed<OP, 8>(calls, splits, n, g);
  }
}

int FLAGCX_CAT(launchReduceGated_, FLAGCX_DT)(const ReduceCall *calls, int n, const GateArgs &g) {
  if (n <= 0) return 0;
  switch (calls[0].op) {
    case kSum: return launchGatedOp<kSum>(calls, n, g);
    case kProd: return launchGatedOp<kProd>(calls, n, g);
    case kMax: return launchGatedOp<kMax>(calls, n, g);
    case kMin: return launchGatedOp<kMin>(calls, n, g);
    case kAvg: return launchGatedOp<kAvg>(calls, n, g);
    default: return (int)hipErrorInvalidValue;
  }
}

// Sums whose member list holds all-zero members that are not read: floating-point types
// add +0.0 once (kSumZ); for integers the sum of the members read is already the result.
#if FLAGCX_DT >= 6
#define FLAGCX_SUM_WITH_ZEROS kSumZ
#else
#define FLAGCX_SUM_WITH_ZEROS kSum
#endif

// n reductions that share k, op and stream.
int FLAGCX_CAT(launchReduceBatch_, FLAGCX_DT)(const ReduceCall *calls, int n) {
  if (n <= 0) return 0;
  if (calls[0].plusZero) return calls[0].op == kSum ? launchBatchOp<FLAGCX_SUM_WITH_ZEROS>(calls, n) : (int)hipErrorInvalidValue;
  switch (calls[0].op) {
    case kSum: return launchBatchOp<kSum>(calls, n);
    case kProd: return launchBatchOp<kProd>(calls, n);
    case kMax: return launchBatchOp<kMax>(calls, n);
    case kMin: return launchBatchOp<kMin>(calls, n);
    case kAvg: return launchBatchOp<kAvg>(calls, n);
    default: return (int)hipErrorInvalidValue;
  }
}

// The resident queue consumer.  Its grid must be resident all at once, so the
// size comes from the occupancy query for this very kernel and LDS reservation.
template <int OP, bool AHEAD>
static int launchQueueOpT(const QueueKernelArgs &q, int wavesPerCU, int numCU, int lds, unsigned maxGrid,
                         hipStream_t stream, unsigned *grid) {
  int fit = 0;
  hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&fit, reduceQueueKernel<elem_t, OP, AHEAD>, 64, (size_t)lds);
  if (e != hipSuccess) return (int)e;
  if (wavesPerCU > 0 && fit > wavesPerCU) fit = wavesPerCU;
  // LDS is handed out in 1280-byte granules on gfx950 (160 KiB per CU): count what
  // really fits, a workgroup that never becomes resident would stall the queue
  if (lds > 0) {
    const int granules = (lds + 1279) / 1280;
    const int byLds = (160 * 1024 / 1280) / granules;
    if (fit > byLds) fit = byLds;
  }
  if (fit < 1) return (int)hipErrorLaunchOutOfResources;
  uint64_t g = (uint64_t)fit * (uint64_t)numCU;
  if (g > maxGrid) g = maxGrid;
  if (g < 2) return (int)hipErrorLaunchOutOfResources;
  *grid = (unsigned)g;
  // workgroups 8n..8n+7 (one per XCD) share ticket counter n modulo the number of
  // counters; every counter in use has workers
  QueueKernelArgs a = q;
  const uint64_t groups = (g - 1) / 8 + 1;
  a.counters = (uint32_t)(groups < (uint64_t)kQueueMaxTicketCounters ? groups : (uint64_t)kQueueMaxTicketCounters);
  reduceQueueKernel<elem_t, OP, AHEAD><<<dim3((unsigned)g), dim3(64), lds, stream>>>(a);
  return (int)hipGetLastError();
}

template <int OP>
static int launchQueueOp(const QueueKernelArgs &q, int wavesPerCU, int numCU, int lds, unsigned maxGrid,
                         hipStream_t stream, unsigned *grid) {
  return q.drawAhead ? launchQueueOpT<OP, true>(q, wavesPerCU, numCU, lds, maxGrid, stream, grid)
                     : launchQueueOpT<OP, false>(q, wavesPerCU, numCU, lds, maxGrid, stream, grid);
}

int FLAGCX_CAT(launchReduceQueue_, FLAGCX_DT)(int op, const QueueKernelArgs &q, int wavesPerCU, int numCU, int lds,
                                              unsigned maxGrid, hipStream_t stream, unsigned *grid) {
  switch (op) {
    case kSum: return launchQueueOp<kSum>(q, wavesPerCU, numCU, lds, maxGrid, stream, grid);
    case kProd: return launchQueueOp<kProd>(q, wavesPerCU, numCU, lds, maxGrid, stream, grid);
    case kMax: return launchQueueOp<kMax>(q, wavesPerCU, numCU, lds, maxGrid, stream, grid);
    case kMin: return launchQueueOp<kMin>(q, wavesPerCU, numCU, lds, maxGrid, stream, grid);
    case kAvg: return launchQueueOp<kAvg>(q, wavesPerCU, numCU, lds, maxGrid, stream, grid);
    default: return (int)hipErrorInvalidValue;
  }
}

int FLAGCX_CAT(launchReduce_, FLAGCX_DT)(const ReduceCall &c) {
  if (c.plusZero) return c.op == kSum ? launchOp<FLAGCX_SUM_WITH_ZEROS>(c) : (int)hipErrorInvalidValue;
  switch (c.op) {
    case kSum: return launchOp<kSum>(c);
    case kProd: return launchOp<kProd>(c);
    case kMax: return launchOp<kMax>(c);
    case kMin: return launchOp<kMin>(c);
    case kAvg: return launchOp<kAvg>(c);
    default: return (int)hipErrorInvalidValue;
  }
}

} // namespace flagcx_amd
