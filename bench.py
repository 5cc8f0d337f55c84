#!/usr/bin/env python3
"""Benchmark of the local N-way reduce and chunk movers on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]          the driver's line
    python bench.py --table sweep|sweep-rotate|configs|dtypes|stride [...]   tables only

One "step" is one pass of the hot path over one batch: a single 8-input bf16 sum
(fp32 accumulation) over 256 MiB per input buffer, i.e. one simulated rank's
reducescatter stage of an 8-rank C2C allreduce.  Inputs are resident in HBM before
the timed region.  Prints ONE JSON line on stdout:

  value      algorithmic bytes / wall time of the K timed steps, GB/s
             ((k+1) * n * sizeof(bf16) per step)
  roofline   the same bytes over the kernel's average launch duration measured
             with HIP events on the launch stream, against 8 TB/s of HBM3E
  configs    the other benchmark configurations, each with its algorithmic bytes,
             ms per pass, GB/s and fraction of the HBM peak: C1 (2 x fp32 sum, 64 MiB),
             C3 (fp16 avg reduce-scatter shard: fused, one batch of 32 chunks, the same
             batch launched up front and opened chunk by chunk, chunk
             by chunk through the reduce queue, 32 chunk launches), C4 (4 x int32
             max / min), C5 (2-input sum, pack, unpack at 4 KiB, 64 MiB, 1 GiB)
  cpu_baseline  the CPU oracle (a port of the reference's host reduce) timed on
             this machine's cores on a bounded sample of the headline workload, and
             the reference's own host path for C1 (its ring all-reduce of two ranks:
             one sum<float> per rank over half the vector), through the library built
             from the reference's templates where that exists
  latency_us_4KiB  per-launch time of a 2-input fp32 sum over 4 KiB buffers

Everything on the GPU goes through the C ABI of libflagcx_amd.so; the oracle is
used only for the cpu_baseline leg and spot checks of results.

Tables (human-readable, no JSON line; the summaries under profiles/ come from them):
  --table sweep         C5: 1 KiB .. 1 GiB, 2-input fp32 sum, pack, unpack, copy, fill
  --table sweep-rotate  the same over several sets of buffers in turn, from --min on
  --table configs       every C1 / C3 / C4 row incl. HIP graph, staging ring, gather
  --table plan          C2C plan replay, literal and fused (--plan-name, --plan-mode, --plan-iters)
  --table dtypes        every element type x operation, --k inputs of --mib MiB
  --table stride        k-input reduce against the inputs' relative placement,
                        wavefronts per CU and inputs in flight
"""
import argparse
import ctypes as C
import json
import os
import sys
import threading
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
K = 8
N_ELEM = 128 * 1024 * 1024          # 256 MiB of bf16 per input
ALGO_BYTES = (K + 1) * N_ELEM * 2   # k reads + 1 write
MiB = 1 << 20

# HBM bytes per launch of the headline kernel from two rocprofv3 --pmc runs
# (FETCH_SIZE, WRITE_SIZE), each scaled by what the same counter reads for a copy of
# known size; not measured by this program.
TRAFFIC_SOURCE = "profiles/reduce8_bf16_sum_256MiB_pmc.txt"
TRAFFIC_BYTES = 2415742177


def log(*a):
    print(*a, file=sys.stderr, flush=True)


# --------------------------------------------------------------------- timing

def timed_ms(fn, warmup=5, iters=20):
    """ms per call of `iters` back-to-back calls (HIP events on the current stream)."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def timed_sets_ms(fn, nsets, warmup=None, iters=20):
    """The same with fn(i) cycling through nsets sets of buffers."""
    import torch
    for i in range(warmup if warmup is not None else max(5, nsets)):
        fn(i % nsets)
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(iters):
        fn(i % nsets)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters


def single_launch_us(fn, nsets=1, warmup=5, iters=20):
    """(median, min) microseconds of single launches, each between its own event pair."""
    import torch
    for i in range(max(warmup, nsets)):
        fn(i % nsets)
    torch.cuda.synchronize()
    ts = []
    for i in range(iters):
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        fn(i % nsets)
        e1.record()
        e1.synchronize()
        ts.append(e0.elapsed_time(e1) * 1e3)
    ts.sort()
    return ts[len(ts) // 2], ts[0]


def row(nbytes, ms, **extra):
    gbps = nbytes / (ms * 1e-3) / 1e9
    r = {"bytes": int(nbytes), "ms": round(ms, 5), "gbps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}
    r.update(extra)
    return r


def placed(L, count, nelem, dtype, separate=False):
    """`count` tensors of nelem elements inside one allocation, at the addresses
    flagcxLocalPlaceBuffers gives (different HBM channel groups); the pool is returned
    too so that it stays alive.  separate: plain torch allocations instead."""
    import torch
    if separate:
        return [torch.empty(nelem, dtype=dtype, device="cuda") for _ in range(count)], None
    esz = torch.empty(0, dtype=dtype).element_size()
    nbytes = nelem * esz
    pool_bytes = count * (nbytes + 128 * 1024)
    pool = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
    base = pool.data_ptr()
    return [pool[a - base: a - base + nbytes].view(dtype) for a in L.place_buffers(base, pool_bytes, nbytes, count)], pool


# --------------------------------------------------------------- CPU baselines

def cpu_headline(inputs_bits, sample_elems):
    """The oracle on a leading sample of the headline inputs (host copies)."""
    from oracle import cpu_oracle as O
    host = [np.ascontiguousarray(t[:sample_elems].cpu().numpy().view(np.uint16)) for t in inputs_bits]
    dst = np.empty(sample_elems, dtype=np.uint16)
    nbytes = (K + 1) * sample_elems * 2
    t1 = O.time_reduce(host, dst, O.BF16, O.SUM, nthreads=1, warmup=1, iters=3)
    ncores = os.cpu_count() or 1
    nth = min(K, ncores)
    tk = O.time_reduce(host, dst, O.BF16, O.SUM, nthreads=nth, warmup=1, iters=3)
    return {
        "value": round(nbytes / t1 / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
        "sample": "first %d of %d elements of the same 8 bf16 inputs (%.0f MiB per input), "
                  "median of 3 passes after 1 warm-up; restatement extension: the reference's "
                  "host path rejects bf16" % (sample_elems, N_ELEM, sample_elems * 2 / 2**20),
        "threads_k": {"value": round(nbytes / tk / 1e9, 3), "threads": nth},
        "host_cores": ncores,
    }, host, dst


def cpu_c1_reference_path():
    """C1 the way the reference runs it on the host: a ring all-reduce of two ranks
    (flagcx/service/bootstrap.cc:702-749) cuts the 64 MiB vector into two 32 MiB
    chunks and each rank folds one of them with ONE sum<float>(res = partial,
    op1 = local, op2 = partial) (bootstrap.cc:651-653).  Timed through the library
    built from the reference's own templates when it is there, through the oracle's
    restatement otherwise; sockets and PCIe copies of that path are left out."""
    from oracle import cpu_oracle as O
    n = 16 * 1024 * 1024
    rng = np.random.default_rng(0)
    a = rng.uniform(-1, 1, n).astype(np.float32)     # in0, then in1, one generator
    b = rng.uniform(-1, 1, n).astype(np.float32)
    half = n // 2
    ref = O.ref_lib()
    kind = "reference" if ref is not None else "port"

    def fold(local, partial):
        # data_for_recv = sum(sendbuff + offset, data_for_recv)
        if ref is not None:
            rc = ref.ref_binary(O.SUM, O.FP32, partial.ctypes.data, local.ctypes.data, partial.ctypes.data, partial.size)
        else:
            rc = O.lib().oracle_binary(O.SUM, O.FP32, partial.ctypes.data, local.ctypes.data, partial.ctypes.data,
                                       partial.size, 1)
        assert rc == 0

    evict = np.zeros(96 * 1024 * 1024, dtype=np.float32)     # 384 MiB: larger than the host's caches

    def one_pass(threads):
        # rank 0 ends with chunk 0 = in1[0:half] (received) + in0[0:half] (local); rank 1 with chunk 1
        p0, p1 = b[:half].copy(), a[half:].copy()
        # the reference's partial arrives over a socket, not from a copy made a moment ago: walk
        # another buffer so that nothing of the operands is left in the caches when the fold starts
        evict.__iadd__(1.0)
        jobs = [(a[:half], p0), (b[half:], p1)]
        t0 = time.perf_counter()
        if threads == 1:
            for loc, par in jobs:
                fold(loc, par)
        else:
            th = [threading.Thread(target=fold, args=j) for j in jobs]
            for t in th:
                t.start()
            for t in th:
                t.join()
        return time.perf_counter() - t0, p0, p1

    res = {}
    for threads in (1, 2):
        one_pass(threads)
        ts = sorted(one_pass(threads)[0] for _ in range(5))
        res[threads] = ts[len(ts) // 2]
    _, p0, p1 = one_pass(1)
    want = a + b
    ok = bool(np.array_equal(np.concatenate([p0, p1]), want))
    nbytes = 3 * n * 4
    return {
        "config": "C1: 2-input fp32 sum, 64 MiB per buffer, uniform[-1,1) seed 0, as the reference's 2-rank host "
                  "ring all-reduce folds it (two sum<float> calls over 8 Mi elements each)",
        "value": round(nbytes / res[1] / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": kind,
        "sample": "the whole configuration (192 MiB of traffic), median of 5 passes after 1 warm-up; operands evicted "
                  "from the host's caches before every timed fold (a 384 MiB buffer is walked in between)",
        "threads_2": {"value": round(nbytes / res[2] / 1e9, 3), "threads": 2,
                      "note": "one thread per simulated rank, each folding its own chunk"},
        "result_equals_in0_plus_in1": ok,
    }, a, b


# ------------------------------------------------------------- configurations

def config_c1(L, separate=False):
    """2-input fp32 sum, 64 MiB per buffer: over the same three buffers launch after
    launch (they fit the 256 MB memory-side cache), over rotating sets, and as the
    reference's ring all-reduce (two chunk folds in one launch)."""
    import torch
    n = 16 * MiB
    nb = 3 * n * 4
    nsets = 9    # 9 x 192 MiB = 1.7 GiB in turn: nothing of a launch's buffers is left in the cache
    sets, keep = [], []
    g = torch.Generator(device="cuda").manual_seed(0)
    for s in range(nsets):
        bufs, pool = placed(L, 3, n, torch.float32, separate)
        keep.append(pool)
        if s == 0:
            bufs[0].copy_(torch.rand(n, generator=g, device="cuda") * 2 - 1)
            bufs[1].copy_(torch.rand(n, generator=g, device="cuda") * 2 - 1)
        else:
            bufs[0].copy_(sets[0][0])
            bufs[1].copy_(sets[0][1])
        sets.append(bufs)
    a, b, out = sets[0]
    out_rows = {}
    ms = timed_ms(lambda: L.reduce([a, b], out, L.RedOp.Sum))
    out_rows["C1_same_buffers"] = row(nb, ms, note="192 MiB working set: inside the 256 MB memory-side cache")
    ms = timed_sets_ms(lambda i: L.reduce(sets[i][:2], sets[i][2], L.RedOp.Sum), nsets)
    out_rows["C1_rotating_buffers"] = row(nb, ms, sets=nsets)
    ms = timed_ms(lambda: L.all_reduce([a, b], out, L.RedOp.Sum))
    out_rows["C1_ring_allreduce"] = row(nb, ms, note="chunk table of the reference's ring: two 32 MiB chunks, one launch")
    ms = timed_sets_ms(lambda i: L.all_reduce(sets[i][:2], sets[i][2], L.RedOp.Sum), nsets)
    out_rows["C1_ring_allreduce_rotating"] = row(nb, ms, sets=nsets)
    return out_rows, (a, b, out)


def make_c3(L, separate=False):
    """8 ranks x 1 GiB fp16, N(0, sigma = 0.01) seeded per rank; shard = 128 MiB."""
    import torch
    nranks, per_rank = 8, 512 * MiB
    shard = per_rank // nranks
    send, pool = placed(L, nranks, per_rank, torch.float16, separate)
    for r in range(nranks):
        g = torch.Generator(device="cuda").manual_seed(100 + r)
        for s in range(nranks):
            send[r][s * shard:(s + 1) * shard] = (torch.randn(shard, generator=g, device="cuda") * 0.01).to(torch.float16)
    recv = torch.empty(shard, dtype=torch.float16, device="cuda")
    return nranks, per_rank, shard, send, recv, pool


def c3_chunk_descs(L, nranks, shard, send, recv, rank):
    chunk_elems = L.CHUNKSIZE // 2
    descs = []
    for c in range(shard // chunk_elems):
        srcs = [send[(rank + 1 + j) % nranks].data_ptr() + (rank * shard + c * chunk_elems) * 2 for j in range(nranks)]
        descs.append((srcs, recv.data_ptr() + c * chunk_elems * 2, chunk_elems))
    return descs


def c3_queue_ms(L, nranks, descs, warmup=5, iters=20):
    """The shard chunk by chunk through the resident reduce queue.  Returns (ms per shard when
    `iters` shards are enqueued back to back and the last ticket is waited for, as the other rows
    are timed; median ms of one shard alone, first enqueue -> return of Wait; resident wavefronts;
    ms of one 4 KiB entry, enqueue -> Wait)."""
    import torch
    lib = L.lib()
    fifo = L.ReduceFifo(64, nranks, L.DataType.Float16, L.RedOp.Avg)
    arrs = [((C.c_void_p * nranks)(*d[0]), d[1], d[2]) for d in descs]
    ticket = C.c_uint64()
    enq = lib.flagcxLocalReduceFifoEnqueueReduce
    times = []
    torch.cuda.synchronize()
    lib.flagcxLocalSetMaxSpinCount(1 << 22)

    def shard():
        for srcs, dst, cnt in arrs:
            while True:
                rc = enq(fifo._h, srcs, nranks, dst, cnt, C.byref(ticket))
                if rc != L.Result.InProgress:
                    break
            fifo._check(rc)

    try:
        with fifo:
            for it in range(warmup + iters):
                t0 = time.perf_counter()
                shard()
                fifo.wait(ticket.value)
                if it >= warmup:
                    times.append((time.perf_counter() - t0) * 1e3)
            t0 = time.perf_counter()
            for it in range(iters):
                shard()
            fifo.wait(ticket.value)
            steady = (time.perf_counter() - t0) * 1e3 / iters
            grid = fifo.grid()
            # what a shard's wall clock holds beside the folding itself: one 4 KiB entry, enqueue -> Wait
            small = []
            for it in range(30):
                t0 = time.perf_counter()
                fifo._check(enq(fifo._h, arrs[0][0], nranks, arrs[0][1], 2048, C.byref(ticket)))
                fifo.wait(ticket.value)
                small.append((time.perf_counter() - t0) * 1e3)
            small.sort()
    finally:
        fifo.close()
        lib.flagcxLocalSetMaxSpinCount(-1)
    times.sort()
    return steady, times[len(times) // 2], grid, small[len(small) // 2]


def c3_gated_ms(L, nranks, descs, warmup=5, iters=20):
    """The shard as ONE batch launched before any chunk is said to be there, its descriptors opened
    chunk by chunk.  Returns (ms per shard when `iters` shards are launched and opened back to back
    with one synchronisation at the end, as the other rows are timed; median ms of one shard alone by
    the host's clock, launch call -> end of the stream synchronisation; the same between two events on
    the launch's stream)."""
    import torch
    lib = L.lib()
    keep = [(C.c_void_p * nranks)(*d[0]) for d in descs]
    arr = (L.ReduceDesc * len(descs))(*[L.ReduceDesc(keep[i], d[1], d[2]) for i, d in enumerate(descs)])
    first = C.c_uint64()
    side = torch.cuda.Stream()
    st = L.Stream(side.cuda_stream)
    times, dev = [], []
    torch.cuda.synchronize()
    lib.flagcxLocalSetMaxSpinCount(1 << 22)
    gate = L.Gate()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)

    def shard():
        L.check(lib.flagcxLocalReduceBatchGated(gate._h, arr, len(descs), nranks, int(L.DataType.Float16),
                                                int(L.RedOp.Avg), C.byref(st), C.byref(first)))
        for c in range(len(descs)):
            lib.flagcxLocalGateOpen(gate._h, first.value + c + 1)

    try:
        for it in range(warmup + iters):
            t0 = time.perf_counter()
            e0.record(side)
            shard()
            e1.record(side)
            side.synchronize()
            if it >= warmup:
                times.append((time.perf_counter() - t0) * 1e3)
                dev.append(e0.elapsed_time(e1))
        t0 = time.perf_counter()
        for it in range(iters):
            shard()
        side.synchronize()
        steady = (time.perf_counter() - t0) * 1e3 / iters
        assert gate.query()[2] == 0, "the gated launch gave up waiting"
    finally:
        gate.destroy()
        lib.flagcxLocalSetMaxSpinCount(-1)
    times.sort()
    dev.sort()
    return steady, times[len(times) // 2], dev[len(dev) // 2]


def config_c3(L, full=False, separate=False):
    import torch
    nranks, per_rank, shard, send, recv, pool = make_c3(L, separate)
    rank = 3
    nb = 9 * shard * 2
    rows = {}
    ms = timed_ms(lambda: L.reduce_scatter(send, rank, recv, L.RedOp.Avg))
    rows["C3_fused"] = row(nb, ms, note="one launch for the 128 MiB shard")
    descs = c3_chunk_descs(L, nranks, shard, send, recv, rank)
    ms = timed_ms(lambda: L.reduce_batch(descs, L.RedOp.Avg, L.DataType.Float16, nranks))
    rows["C3_batch_32x4MiB"] = row(nb, ms, note="32 chunk descriptors, one batch call (needs every chunk present)")
    frac_of = lambda t: round(nb / (t * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4)
    try:
        ms, single, grid, small_ms = c3_queue_ms(L, nranks, descs)
        rows["C3_queue_32x4MiB"] = row(nb, ms, note="chunk by chunk through the resident reduce queue: 20 shards enqueued back "
                                                    "to back, host wall clock to the return of Wait on the last ticket, per "
                                                    "shard; %d resident wavefronts" % grid,
                                       one_shard_enqueue_to_wait_ms=round(single, 5), one_shard_frac=frac_of(single),
                                       one_4KiB_entry_enqueue_to_wait_ms=round(small_ms, 5))
    except Exception as e:   # a row of its own: the others are measured all the same
        rows["C3_queue_32x4MiB"] = {"error": repr(e)}
    try:
        ms, single, dev_ms = c3_gated_ms(L, nranks, descs)
        rows["C3_gated_batch_32x4MiB"] = row(nb, ms, note="one batch launched up front, a host store per chunk lets its "
                                                          "wavefronts go: 20 shards launched and opened back to back, host wall "
                                                          "clock to the end of one stream synchronisation, per shard",
                                             one_shard_launch_to_sync_ms=round(single, 5), one_shard_frac=frac_of(single),
                                             one_shard_device_ms=round(dev_ms, 5), one_shard_device_frac=frac_of(dev_ms),
                                             device_note="device: between two events on the launch's stream, recorded before "
                                                         "the launch call and behind the last Open; launch_to_sync also holds "
                                                         "the host's wake-up from the synchronisation (about 10 us)")
    except Exception as e:
        rows["C3_gated_batch_32x4MiB"] = {"error": repr(e)}
    ms = timed_ms(lambda: L.reduce_scatter(send, rank, recv, L.RedOp.Avg, chunkbytes=L.CHUNKSIZE))
    rows["C3_per_chunk_launches"] = row(nb, ms, note="32 launches of 4 MiB chunks on one stream, %.2f us per launch"
                                                     % (ms * 1e3 / 32))
    try:
        # the 7 peers' slices staged through a 16 x 4 MiB ring on a second stream, as the proxies move them
        ring_mem = torch.empty(L.CHUNKSIZE * 16 * (nranks - 1), dtype=torch.uint8, device="cuda")
        ring = L.Ring(ring_mem, nranks - 1)
        copy_t = torch.cuda.Stream()
        staged = nb + 2 * (nranks - 1) * shard * 2
        ms = timed_ms(lambda: ring.reduce_scatter(send, rank, recv, L.RedOp.Avg, L.Stream(copy_t.cuda_stream),
                                                  L.current_stream()))
        rows["C3_staging_ring_2_streams"] = row(nb, ms, hbm_bytes_incl_staging=staged,
                                                hbm_gbps=round(staged / ms / 1e6, 1),
                                                hbm_frac=round(staged / ms / 1e6 / HBM_PEAK_GBPS, 4),
                                                note="every peer slice is copied into a ring slot and read again by the "
                                                     "reduce: 2.56 x the bytes of the fold alone")
        ring.close()
        del ring_mem
    except Exception as e:
        rows["C3_staging_ring_2_streams"] = {"error": repr(e)}
    if full:
        # the 32 chunk launches captured once into a HIP graph and replayed
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            L.reduce_scatter(send, rank, recv, L.RedOp.Avg, chunkbytes=L.CHUNKSIZE)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            L.reduce_scatter(send, rank, recv, L.RedOp.Avg, chunkbytes=L.CHUNKSIZE)
        rows["C3_per_chunk_launches_hip_graph"] = row(nb, timed_ms(graph.replay))
        del graph
        ring_mem = torch.empty(L.CHUNKSIZE * 16 * (nranks - 1), dtype=torch.uint8, device="cuda")
        ring = L.Ring(ring_mem, nranks - 1)
        copy_t = torch.cuda.Stream()
        cs = L.Stream(copy_t.cuda_stream)
        staged = nb + 2 * (nranks - 1) * shard * 2
        L.lib().flagcxLocalSetMaxSpinCount(1 << 22)
        fifo = L.ReduceFifo(64, nranks, L.DataType.Float16, L.RedOp.Avg)
        # a hardware queue of its own for the consumer: the copy stream must never wait behind it
        fifo.set_own_queue(True)
        torch.cuda.synchronize()
        with fifo:
            for _ in range(5):
                ring.reduce_scatter_fifo(fifo, send, rank, recv, cs)
            t0 = time.perf_counter()
            for _ in range(20):
                ring.reduce_scatter_fifo(fifo, send, rank, recv, cs)
            ms = (time.perf_counter() - t0) * 1e3 / 20
        fifo.close()
        L.lib().flagcxLocalSetMaxSpinCount(-1)
        rows["C3_staging_ring_polled_into_queue"] = row(nb, ms, hbm_bytes_incl_staging=staged,
                                                        hbm_gbps=round(staged / ms / 1e6, 1))
        ring.close()
        del ring_mem

        def all_shards():
            for rk in range(nranks):
                L.reduce_scatter(send, rk, recv, L.RedOp.Avg)
        rows["C3_all_8_shards"] = row(8 * nb, timed_ms(all_shards, warmup=2, iters=5))
        # The stage after it in an all-reduce: every rank holds one reduced slice in a buffer of
        # the full size.  The reference zero-fills the rest of each buffer and sum-all-reduces the
        # buffers (flagcx/core/c2c_algo.cc:586-608 + :310-336); slice copies do the same job.
        fullbuf = torch.empty(per_rank, dtype=torch.float16, device="cuda")

        def refresh_and_sum():
            for rk in range(nranks):
                L.refresh(send[rk], 0, rk * shard, shard, per_rank, L.RedOp.Sum)
            L.reduce(send, fullbuf, L.RedOp.Sum)
        traffic = nranks * (per_rank - shard) * 2 + (nranks + 1) * per_rank * 2
        rows["C3_gather_zero_fill_plus_sum"] = row(traffic, timed_ms(refresh_and_sum, warmup=2, iters=5))

        def copy_slices():
            for rk in range(nranks):
                L.memcpy(fullbuf.data_ptr() + rk * shard * 2, send[rk].data_ptr() + rk * shard * 2, shard * 2)
        rows["C3_gather_8_slice_copies"] = row(2 * per_rank * 2, timed_ms(copy_slices, warmup=2, iters=5))
        del fullbuf
    del send, recv, pool
    torch.cuda.empty_cache()
    return rows


def config_c4(L, separate=False):
    import torch
    n = 128 * MiB
    g = torch.Generator(device="cuda").manual_seed(3)
    bufs, pool = placed(L, 5, n, torch.int32, separate)
    ins, out = bufs[:4], bufs[4]
    for t in ins:
        t.copy_(torch.randint(-2**31, 2**31 - 1, (n,), generator=g, device="cuda", dtype=torch.int32))
    rows = {}
    for op, nm in ((L.RedOp.Max, "max"), (L.RedOp.Min, "min")):
        rows["C4_" + nm] = row(5 * n * 4, timed_ms(lambda: L.reduce(ins, out, op)))
    del bufs, pool
    torch.cuda.empty_cache()
    return rows


def config_headline_variants(L, inputs):
    """The headline fold under three conditions a caller may bring: nine ordinary allocations
    (whatever addresses the allocator gives), sources two bytes further on than the destination
    (chunk offsets are elemOffset * dtypeSize, flagcx/core/c2c_algo.cc:313-316, so sources need
    not agree with the destination modulo 16), and sixteen inputs."""
    import torch
    rows = {}
    n = N_ELEM
    try:
        bufs = [torch.empty(n, dtype=torch.bfloat16, device="cuda") for _ in range(K + 1)]
        for j in range(K):
            bufs[j].copy_(inputs[j])
        ms = timed_ms(lambda: L.reduce(bufs[:K], bufs[K], L.RedOp.Sum))
        rows["headline_allocator_layout"] = row(ALGO_BYTES, ms, note="nine separate torch allocations instead of "
                                                                      "buffers placed by flagcxLocalPlaceBuffers")
        del bufs
        torch.cuda.empty_cache()
    except Exception as e:
        rows["headline_allocator_layout"] = {"error": repr(e)}
    try:
        pools, pool = placed(L, K + 1, n + 8, torch.bfloat16)
        srcs = [pools[j][1:n + 1] for j in range(K)]            # + 2 bytes
        dst = pools[K][:n]
        for j in range(K):
            srcs[j].copy_(inputs[j])
        ms = timed_ms(lambda: L.reduce(srcs, dst, L.RedOp.Sum))
        rows["headline_sources_plus_2_bytes"] = row(ALGO_BYTES, ms, note="every source 2 bytes past a 16-byte line, the "
                                                                          "destination on one: aligned loads and lane shifts")
        del pools, pool, srcs, dst
        torch.cuda.empty_cache()
    except Exception as e:
        rows["headline_sources_plus_2_bytes"] = {"error": repr(e)}
    try:
        k16 = 16
        bufs, pool = placed(L, k16 + 1, n, torch.bfloat16)
        for j in range(k16):
            bufs[j].copy_(inputs[j % K])
        ms = timed_ms(lambda: L.reduce(bufs[:k16], bufs[k16], L.RedOp.Sum), warmup=3, iters=10)
        rows["K16_bf16_sum_256MiB"] = row((k16 + 1) * n * 2, ms, note="sixteen inputs: two batches of eight loads, "
                                                                      "accumulators kept in registers")
        del bufs, pool
        torch.cuda.empty_cache()
    except Exception as e:
        rows["K16_bf16_sum_256MiB"] = {"error": repr(e)}
    return rows


def config_plan_replay(L, mib=128, iters=10, only=None, modes=(False, True)):
    """C2C plan replay: the plan documents under tests/golden/plans (written by the reference's
    plan DSL) replayed for all ranks on this GPU, the literal way (every refresh a zero-fill, every
    collective reads all members) and the fused way (sums read the members that hold data).
    `bytes` of both rows of a pair = the algorithmic bytes of the fused replay, i.e. what has to
    move; `issued_bytes` = what that replay handed to the kernels."""
    import torch
    plans = os.path.join(ROOT, "tests", "golden", "plans")
    rows = {}
    cl8 = [0, 0, 0, 0, 1, 1, 1, 1]
    n = mib * MiB // 4
    for name, commop, scratch, algo in (("allreduce8", 6, False, 2), ("reducescatter8", 8, True, 0)):
        if only and name != only:
            continue
        try:
            send = [torch.empty(n, dtype=torch.float32, device="cuda").uniform_(-1, 1) for _ in range(8)]
            recv = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(8)]
            scr = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(8)] if scratch else None
            res, outs = {}, {}
            for fused in modes:
                plan = L.Plan(cl8, n, commop, L.RedOp.Sum)
                plan.set_chunks(8)
                plan.import_xml(os.path.join(plans, name))
                plan.set_algorithm(algo)
                plan.set_fused(fused)
                args = ([t.data_ptr() for t in send], [t.data_ptr() for t in recv],
                        [t.data_ptr() for t in scr] if scr else None, int(L.DataType.Float32))
                ms = timed_ms(lambda: plan.execute(*args), warmup=2, iters=iters)
                res[fused] = (ms,) + plan.traffic()
                outs[fused] = [t[:n // 8 if commop == 8 else n].clone() for t in recv]
                plan.close()
            if len(res) < 2:      # one mode only (profiling runs): its own bytes
                for fused, (ms, issued, launches) in res.items():
                    rows["plan_%s_%s" % (name, "fused" if fused else "literal")] = row(issued, ms, launches=int(launches))
                continue
            same = all(torch.equal(a.view(torch.int32), b.view(torch.int32)) for a, b in zip(outs[False], outs[True]))
            need = res[True][1]
            for fused, tag in ((False, "literal"), (True, "fused")):
                ms, issued, launches = res[fused]
                rows["plan_%s_%s" % (name, tag)] = row(need, ms, issued_bytes=int(issued), launches=int(launches),
                                                       issued_gbps=round(issued / ms / 1e6, 1),
                                                       issued_frac=round(issued / ms / 1e6 / HBM_PEAK_GBPS, 4))
            rows["plan_%s_fused" % name]["same_bytes_as_literal"] = bool(same)
            rows["plan_%s_fused" % name]["speedup_over_literal"] = round(res[False][0] / res[True][0], 3)
            rows["plan_%s_literal" % name]["note"] = (
                "8 ranks x %d MiB fp32, 2 clusters of 4, plan %s (algorithm %d)%s; bytes = what the fused replay moves"
                % (mib, name, algo, ", scratch per rank" if scratch else ""))
            del send, recv, scr, outs
            torch.cuda.empty_cache()
        except Exception as e:
            rows["plan_%s_error" % name] = repr(e)
    return rows


def config_fanout(L, mib=256, ndst=4):
    """One source to `ndst` destinations (a broadcast inside a simulated cluster): flagcxLocalCopyFanout reads
    the source once, (1 + n) bytes per payload byte; beside it the same copies as one batch launch, 2 n."""
    import torch
    rows = {}
    try:
        n = mib * MiB
        sets = []
        for _ in range(2):
            src = torch.empty(n, dtype=torch.uint8, device="cuda")
            src.random_(0, 255)
            sets.append((src, [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(ndst)]))

        def fan(i):
            s, d = sets[i]
            L.copy_fanout([(s.data_ptr(), [x.data_ptr() for x in d], n)])

        def one_by_one(i):
            s, d = sets[i]
            L.reduce_batch([([s.data_ptr()], x.data_ptr(), n) for x in d], L.RedOp.Sum, L.DataType.Uint8, 1)
        ms_f = timed_sets_ms(fan, 2, warmup=4, iters=20)
        ok = all(torch.equal(sets[0][0], x) for x in sets[0][1])
        ms_c = timed_sets_ms(one_by_one, 2, warmup=4, iters=20)
        rows["fanout_1_to_%d_%dMiB" % (ndst, mib)] = row((1 + ndst) * n, ms_f, destinations_equal_source=bool(ok),
                                                        speedup_over_separate_copies=round(ms_c / ms_f, 3))
        rows["copies_%dx_%dMiB_one_batch" % (ndst, mib)] = row(2 * ndst * n, ms_c)
        del sets
        torch.cuda.empty_cache()
    except Exception as e:
        rows["fanout_error"] = repr(e)
    return rows


def plan_replay_small(L, sizes_kib=(64, 1024, 8192), iters=50):
    """Small collectives are bound by the launches of a replay, not by bytes.  flagcxLocalPlanExecute
    only launches kernels, so one Execute captured into a HIP graph stands for every later one with
    the same buffers: microseconds per fused replay of the allreduce8 plan, eager and from a graph."""
    import torch
    plans = os.path.join(ROOT, "tests", "golden", "plans")
    cl8 = [0, 0, 0, 0, 1, 1, 1, 1]
    rows = {}
    for kib in sizes_kib:
        try:
            n = kib * 1024 // 4
            send = [torch.empty(n, dtype=torch.float32, device="cuda").uniform_(-1, 1) for _ in range(8)]
            recv = [torch.empty(n, dtype=torch.float32, device="cuda") for _ in range(8)]
            plan = L.Plan(cl8, n, 6, L.RedOp.Sum)
            plan.set_chunks(8)
            plan.import_xml(os.path.join(plans, "allreduce8"))
            plan.set_algorithm(2)
            args = ([t.data_ptr() for t in send], [t.data_ptr() for t in recv], None, int(L.DataType.Float32))
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                eager_ms = timed_ms(lambda: plan.execute(*args), warmup=5, iters=iters)
                want = [t.clone() for t in recv]
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g, stream=side, capture_error_mode="global"):
                    plan.execute(*args)
                for t in recv:
                    t.zero_()
                graph_ms = timed_ms(g.replay, warmup=5, iters=iters)
                same = all(torch.equal(a.view(torch.int32), b.view(torch.int32)) for a, b in zip(want, recv))
            issued, launches = plan.traffic()
            rows["plan_allreduce8_fused_%dKiB" % kib] = {
                "bytes": int(issued), "launches": int(launches), "eager_us": round(eager_ms * 1e3, 2),
                "graph_us": round(graph_ms * 1e3, 2), "graph_same_bytes_as_eager": bool(same),
                "note": "8 ranks x %d KiB fp32, back-to-back replays between two HIP events" % kib}
            plan.close()
            del g
        except Exception as e:
            rows["plan_allreduce8_fused_%dKiB" % kib] = {"error": repr(e)}
    return rows


def perf_driver(*argv, timeout=180):
    """Lines of flagcx_amd/lib/local_perf (a C++ caller of the C ABI), or None with the reason logged."""
    import subprocess
    perf_bin = os.path.join(ROOT, "flagcx_amd", "lib", "local_perf")
    if not os.path.exists(perf_bin):
        return None
    try:
        r = subprocess.run([perf_bin] + list(argv), capture_output=True, text=True, timeout=timeout)
        if r.returncode != 0:
            log("bench.py: local_perf %s failed (%d): %s" % (" ".join(argv), r.returncode, r.stderr[-300:]))
            return None
        return r.stdout.splitlines()
    except Exception as e:
        log("bench.py: local_perf %s failed: %r" % (" ".join(argv), e))
        return None


def measured_ceiling():
    """What this GPU's memory gives: read-only streams (the reduce kernels' shape without the
    store stream), the library's fill, copy and 8-input sum at the same size, in one process."""
    lines = perf_driver("-C", "1")
    if not lines:
        return None
    out = {"unit": "GB/s", "bytes_walked_per_probe": 16 << 30,
           "method": "flagcx_amd/lib/local_perf -C 1: bytes moved / time of 10 back-to-back launches between two HIP "
                     "events after 3 warm-up launches, every probe over 16 GiB (64 x the memory-side cache, which holds part "
                     "of a smaller walk whatever its order); the 8-input sum at the headline size over 4 sets of "
                     "buffers; the read-only "
                     "probe has the reduce kernels' shape without the store stream and is swept over 8 caps on resident "
                     "wavefronts and 3 load pacings per stream count, best reported"}
    for l in lines:
        w = l.split()
        if len(w) >= 3 and w[0] == "ceiling":
            out[w[1]] = float(w[2])
            if len(w) > 3:
                out[w[1] + "_shape"] = " ".join(w[3:])
    reads = [v for k, v in out.items() if k.startswith("read_only") and isinstance(v, float)]
    if reads:
        out["best_read_only"] = max(reads)
    return out


def latency_floor():
    lines = perf_driver("-L", "1", "-n", "40")
    if not lines:
        return None
    out = {"columns": "us per call: back to back between two events / one call between its own event pair / "
                      "call -> hipStreamSynchronize / host time of the call while the stream is busy (medians; "
                      "flagcx_amd/lib/local_perf -L 1)"}
    for l in lines:
        w = l.split()
        if len(w) == 6 and w[0] == "floor":
            out[w[1]] = {"back_to_back": float(w[2]), "single_between_events": float(w[3]), "launch_to_sync": float(w[4]),
                         "host_call": float(w[5])}
    if "library_reduce2_fp32" in out:
        for other, key in (("empty_kernel_1x64", "library_above_empty_launch_back_to_back"),
                           ("minimal_sum_kernel_4x64", "library_above_minimal_sum_kernel_back_to_back")):
            if other in out:
                out[key] = round(out["library_reduce2_fp32"]["back_to_back"] - out[other]["back_to_back"], 3)
    return out


def sweep_point(L, size, rotate, g):
    """One size of C5: (nsets, {kernel: (median us, GB/s)}, back-to-back us of the 2-input sum)."""
    import torch
    lib = L.lib()
    st = L.current_stream()
    sref = C.byref(st)
    f32, opsum = int(L.DataType.Float32), int(L.RedOp.Sum)
    n = size // 4
    chunk = size // 8
    nsets = 1
    if rotate:
        nsets = max(2, min(16, ((3 << 29) + 2 * size - 1) // (2 * size)))
    bufs = []
    for _ in range(nsets):
        a = torch.rand(n, device="cuda", generator=g) * 2 - 1
        b = torch.rand(n, device="cuda", generator=g) * 2 - 1
        c = torch.empty(n, device="cuda")
        # sparse source of 8*size bytes holding 8 chunks of size/8 at stride `size`
        sparse = torch.rand(8 * n, device="cuda", generator=g)
        staged = torch.empty(n, device="cuda")
        bufs.append((a, b, c, sparse, staged, (C.c_void_p * 2)(a.data_ptr(), b.data_ptr())))
    fns = {
        "reduce2": (3 * size, lambda i: lib.flagcxLocalReduce(bufs[i][5], 2, bufs[i][2].data_ptr(), n, f32, opsum, sref)),
        "pack": (2 * size, lambda i: lib.flagcxLocalPack(bufs[i][4].data_ptr(), bufs[i][3].data_ptr(), 8, chunk, size, sref)),
        "unpack": (2 * size, lambda i: lib.flagcxLocalUnpack(bufs[i][3].data_ptr(), bufs[i][4].data_ptr(), 8, chunk, size, sref)),
        "memcpy": (2 * size, lambda i: lib.flagcxLocalMemcpy(bufs[i][2].data_ptr(), bufs[i][0].data_ptr(), size, sref)),
        "memset": (size, lambda i: lib.flagcxLocalMemset(bufs[i][2].data_ptr(), 0, size, sref)),
    }
    out = {}
    for name, (nb, fn) in fns.items():
        assert fn(0) == 0, name
        med, _ = single_launch_us(fn, nsets)
        out[name] = (med, nb / med / 1e3, nb)
    nb2b = 1000 if size <= (1 << 20) else 50
    b2b = timed_sets_ms(fns["reduce2"][1], nsets, warmup=20, iters=nb2b) * 1e3
    del bufs
    torch.cuda.empty_cache()
    return nsets, out, b2b


def config_c5(L):
    import torch
    g = torch.Generator(device="cuda").manual_seed(0)
    rows = {}
    for size, name, rotate in ((4096, "C5_4KiB", False), (64 * MiB, "C5_64MiB", True), (1 << 30, "C5_1GiB", True)):
        nsets, out, b2b = sweep_point(L, size, rotate, g)
        r = {"bytes_per_buffer": size, "sets": nsets}
        for k in ("reduce2", "pack", "unpack"):
            med, gbps, nb = out[k]
            r[k] = {"bytes": nb, "us": round(med, 2), "gbps": round(gbps, 1), "frac": round(gbps / HBM_PEAK_GBPS, 4)}
        r["reduce2"]["back_to_back_us"] = round(b2b, 2)
        if size == 4096:
            r["note"] = "launch-latency bound: us per single launch between its own event pair"
        rows[name] = r
    return rows


# --------------------------------------------------------------------- tables

def table_sweep(L, args):
    import torch
    g = torch.Generator(device="cuda").manual_seed(0)
    print("%12s %10s | %9s %9s | %9s %9s | %9s %9s | %9s %9s | %9s %9s | %8s %8s %6s" %
          ("bytes", "sets", "reduce2us", "GB/s", "pack us", "GB/s", "unpack us", "GB/s", "memcpy us", "GB/s",
           "memset us", "GB/s", "b2b us", "b2b GB/s", "% peak"))
    size = args.min
    while size <= args.max:
        nsets, out, b2b = sweep_point(L, size, args.table == "sweep-rotate", g)
        print("%12d %10d | " % (size, nsets) +
              " | ".join("%9.2f %9.1f" % out[k][:2] for k in ("reduce2", "pack", "unpack", "memcpy", "memset")) +
              " | %8.2f %8.1f %6.1f" % (b2b, 3 * size / b2b / 1e3, 3 * size / b2b / 1e3 / HBM_PEAK_GBPS * 100), flush=True)
        size *= 2


def table_configs(L, args):
    rows = {}
    rows.update(config_c1(L, args.allocator_layout)[0])
    rows.update(config_c3(L, full=True, separate=args.allocator_layout))
    rows.update(config_c4(L, args.allocator_layout))
    rows.update(config_fanout(L))
    rows.update(config_plan_replay(L))
    for name, r in rows.items():
        if not isinstance(r, dict) or "bytes" not in r:
            print("%-36s %s" % (name, r), flush=True)
            continue
        extra = "  ".join("%s=%s" % (k, v) for k, v in r.items() if k not in ("bytes", "ms", "gbps", "frac"))
        print("%-36s %14d B  %9.4f ms  %8.1f GB/s  %5.1f %%  %s" % (name, r["bytes"], r["ms"], r["gbps"],
                                                                      100 * r["frac"], extra), flush=True)


def table_plan(L, args):
    """C2C plan replay rows only: --plan-name allreduce8|reducescatter8, --plan-mode literal|fused|both."""
    modes = {"literal": (False,), "fused": (True,), "both": (False, True)}[args.plan_mode]
    rows = config_plan_replay(L, mib=args.mib if args.mib != 256 else 128, iters=args.plan_iters, only=args.plan_name,
                              modes=modes)
    for name, r in rows.items():
        if not isinstance(r, dict) or "bytes" not in r:
            print("%-36s %s" % (name, r), flush=True)
            continue
        extra = "  ".join("%s=%s" % (k, v) for k, v in r.items() if k not in ("bytes", "ms", "gbps", "frac", "note"))
        print("%-32s %14d B  %9.4f ms  %8.1f GB/s  %5.1f %%  %s" % (name, r["bytes"], r["ms"], r["gbps"],
                                                                      100 * r["frac"], extra), flush=True)
    if args.plan_name in (None, "allreduce8") and args.plan_mode == "both":   # one-mode runs are the profiled ones
        for name, r in plan_replay_small(L).items():
            print("%-32s %s" % (name, "  ".join("%s=%s" % kv for kv in r.items() if kv[0] != "note")), flush=True)


def table_fanout(L, args):
    """flagcxLocalCopyFanout, one source of --mib MiB to n destinations, beside the same n copies as one batch
    launch; rotating buffer sets.  --once: one fan-out launch per n and nothing else (for counter runs)."""
    import torch
    n = args.mib * MiB
    print("one source of %d MiB to n destinations; GB/s of (1 + n) x size (fan-out) and of 2 n x size (batch of copies)" % args.mib,
          flush=True)
    for nd in (1, 2, 3, 4, 6, 8):
        sets = []
        for _ in range(1 if args.once else 3):
            src = torch.empty(n, dtype=torch.uint8, device="cuda")
            src.random_(0, 255)
            sets.append((src, [torch.empty(n, dtype=torch.uint8, device="cuda") for _ in range(nd)]))

        def fan(i):
            s, d = sets[i]
            L.copy_fanout([(s.data_ptr(), [x.data_ptr() for x in d], n)])

        def one_by_one(i):
            s, d = sets[i]
            L.reduce_batch([([s.data_ptr()], x.data_ptr(), n) for x in d], L.RedOp.Sum, L.DataType.Uint8, 1)
        if args.once:
            fan(0)
            torch.cuda.synchronize()
            print("  1 -> %d launched once" % nd, flush=True)
        else:
            ms_f = timed_sets_ms(fan, 3, warmup=6, iters=18)
            ms_c = timed_sets_ms(one_by_one, 3, warmup=6, iters=18)
            print("  1 -> %d   fan-out %8.4f ms %7.0f GB/s %5.1f %%    batch of copies %8.4f ms %7.0f GB/s %5.1f %%    %.2f x"
                  % (nd, ms_f, (1 + nd) * n / ms_f / 1e6, (1 + nd) * n / ms_f / 1e6 / 80, ms_c, 2 * nd * n / ms_c / 1e6,
                     2 * nd * n / ms_c / 1e6 / 80, ms_c / ms_f), flush=True)
        del sets
        torch.cuda.empty_cache()


def table_dtypes(L, args):
    import torch
    lib = L.lib()
    names = ["int8", "uint8", "int32", "uint32", "int64", "uint64", "fp16", "fp32", "fp64", "bf16"]
    sizes = [1, 1, 4, 4, 8, 8, 2, 4, 8, 2]
    ops = [("sum", L.RedOp.Sum), ("prod", L.RedOp.Prod), ("max", L.RedOp.Max), ("min", L.RedOp.Min), ("avg", L.RedOp.Avg)]
    nbytes = args.mib * MiB
    st = L.current_stream()
    sref = C.byref(st)
    for k in args.k:
        sets = []
        for _ in range(args.sets):
            pool_bytes = (k + 1) * (nbytes + 128 * 1024)
            pool = torch.empty(pool_bytes, dtype=torch.uint8, device="cuda")
            pool.view(torch.int16).random_(0, 16000)     # finite, normal values in every floating-point type
            addrs = L.place_buffers(pool.data_ptr(), pool_bytes, nbytes, k + 1)
            sets.append(((C.c_void_p * k)(*addrs[:k]), addrs[k], pool))
        print("k=%d, %d MiB per input, %d buffer set(s) in turn; percent of 8 TB/s" % (k, args.mib, args.sets), flush=True)
        for dt in range(10):
            count = nbytes // sizes[dt]
            line = "  %-7s" % names[dt]
            for oname, op in ops:
                def go(i):
                    srcs, dst, _ = sets[i]
                    L.check(lib.flagcxLocalReduce(srcs, k, dst, count, dt, int(op), sref))
                ms = timed_sets_ms(go, args.sets, warmup=2 * args.sets, iters=16)
                line += "  %s %5.1f" % (oname, (k + 1) * nbytes / (ms * 1e-3) / 1e9 / 80.0)
            print(line, flush=True)
        del sets
        torch.cuda.empty_cache()


POSITIONS = [("every buffer on a 128-byte line", lambda j, k: 0, 0),
             ("every buffer 16 bytes into a line", lambda j, k: 16, 16),
             ("every buffer 64 bytes into a line", lambda j, k: 64, 64),
             ("sources 16 bytes in, destination on a line", lambda j, k: 16, 0),
             ("sources on a line, destination 16 bytes in", lambda j, k: 0, 16),
             ("sources 80 bytes in, destination 16 bytes in", lambda j, k: 80, 16),
             ("sources 2..14 bytes in (another offset modulo 16)", lambda j, k: 2 + 2 * (j % 7), 0),
             ("the same, destination 16 bytes in", lambda j, k: 2 + 2 * (j % 7), 16),
             ("every source at a place of its own, dest. on a line", lambda j, k: 16 * ((3 * j) % 8), 0)]


def table_positions(L, args):
    """bf16 sum of k inputs whose buffers start at several positions inside their 128-byte
    cache lines (separate allocations, --sets sets used in turn); percent of 8 TB/s.
    --once: one launch per case and nothing else (for counter runs)."""
    import torch
    lib = L.lib()
    nbytes = args.mib * MiB
    n = nbytes // 2
    st = L.current_stream()
    sref = C.byref(st)
    for k in args.k:
        nsets = 1 if args.once else args.sets
        raws = [[torch.empty(n + 256, dtype=torch.bfloat16, device="cuda") for _ in range(k + 1)] for _ in range(nsets)]
        for raw in raws:
            for t in raw[:k]:
                t.view(torch.int16).random_(0, 16000)
        if not args.once:
            print("k=%d bf16 sum, %d MiB per input, %d buffer set(s) in turn; percent of 8 TB/s" % (k, args.mib, nsets),
                  flush=True)
        for name, so, do in POSITIONS:
            sets = [((C.c_void_p * k)(*[raw[j].data_ptr() + so(j, k) for j in range(k)]), raw[k].data_ptr() + do)
                    for raw in raws]

            def go(i):
                L.check(lib.flagcxLocalReduce(sets[i][0], k, sets[i][1], n, 9, int(L.RedOp.Sum), sref))
            if args.once:
                go(0)
                torch.cuda.synchronize()
                continue
            ms = timed_sets_ms(go, nsets, warmup=2 * nsets, iters=8 * nsets)
            print("  %-52s %5.1f" % (name, (k + 1) * nbytes / (ms * 1e-3) / 1e9 / 80.0), flush=True)
        del raws
        torch.cuda.empty_cache()


STRIDES = [128 * MiB, 128 * MiB + 4096, 128 * MiB + 65536, 129 * MiB + 4096, 256 * MiB, 512 * MiB,
           1024 * MiB, 1024 * MiB + 4096, 1024 * MiB + 65536, 1025 * MiB, 1026 * MiB + 8192, 1057 * MiB + 12288]
CAPS = [8, 10, 12, 14, 16, 18, 21, 25, 0, -1]   # caps that whole LDS granules can express; -1 = the library's choice


def table_stride(L, args):
    """The inputs are slices of one allocation, `stride` bytes apart, so their addresses
    alias differently in the HBM channel hash; per stride, percent of peak for several caps
    on resident wavefronts per CU and for the library's own choice ("auto")."""
    import torch
    lib = L.lib()
    k = args.k[0]
    tdt = torch.bfloat16
    esz = 2
    nbytes = args.mib * MiB
    n = nbytes // esz
    cap0, loads0 = C.c_int(0), C.c_int(0)
    L.check(lib.flagcxLocalGetTune(k, C.byref(cap0)))
    L.check(lib.flagcxLocalGetTuneLoads(k, C.byref(loads0)))
    bigs, outs = [], []
    for _ in range(args.sets):
        big = torch.empty((max(STRIDES) * (k - 1) + nbytes) // esz + 16, dtype=tdt, device="cuda")
        big.view(torch.int16).random_(0, 1000)
        bigs.append(big)
        outs.append(torch.empty(n, dtype=tdt, device="cuda"))
    print("k=%d bf16, %d MiB per input, %d buffer set(s), inputs in flight per wavefront in the cap columns: %s; "
          "percent of 8 TB/s, (k+1)*bytes/time" % (k, args.mib, args.sets, "library's choice" if args.loads < 0 else args.loads))
    print("%14s " % "stride" + " ".join("%7s" % ("cap %d" % c if c > 0 else "no cap" if c == 0 else "auto") for c in CAPS))
    worst = {c: 100.0 for c in CAPS}
    best = {c: 0.0 for c in CAPS}
    try:
        for stv in STRIDES:
            srcs = [[big[j * stv // esz: j * stv // esz + n] for j in range(k)] for big in bigs]
            cells = []
            for cap in CAPS:
                L.check(lib.flagcxLocalTune(k, cap))
                L.check(lib.flagcxLocalTuneLoads(k, args.loads if cap >= 0 else -1))
                ms = timed_sets_ms(lambda i: L.reduce(srcs[i], outs[i], L.RedOp.Sum), args.sets,
                                   warmup=3 * args.sets, iters=20 * args.sets)
                pct = (k + 1) * nbytes / (ms * 1e-3) / 1e9 / 80.0
                worst[cap] = min(worst[cap], pct)
                best[cap] = max(best[cap], pct)
                cells.append("%7.1f" % pct)
            print("%14d " % stv + " ".join(cells), flush=True)
    finally:
        L.check(lib.flagcxLocalTune(k, cap0.value))
        L.check(lib.flagcxLocalTuneLoads(k, loads0.value))
    print("%14s " % "worst..best" + " ".join("%3.0f..%-3.0f" % (worst[c], best[c]) for c in CAPS))


# ----------------------------------------------------------------------- main

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--cpu-sample", type=int, default=32 * 1024 * 1024,
                    help="elements per input the CPU baseline reduces")
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the C1 / C3 / C4 / C5 rows")
    ap.add_argument("--allocator-layout", action="store_true",
                    help="inputs and output as separate torch allocations instead of placed in one")
    ap.add_argument("--rotate-sets", type=int, default=3, metavar="S",
                    help="also time the same launches over S sets of buffers used in turn (0: skip), "
                         "reported as rotating_buffers")
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="N",
                    help="also run N flagcxLocalMemcpy launches of 256 MiB (a copy of known size "
                         "to scale rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    ap.add_argument("--plan-name", default=None, help="plan table: allreduce8 or reducescatter8 (default both)")
    ap.add_argument("--plan-mode", default="both", choices=["literal", "fused", "both"], help="plan table: which replay")
    ap.add_argument("--plan-iters", type=int, default=10, help="plan table: timed replays per row")
    ap.add_argument("--table", choices=["sweep", "sweep-rotate", "configs", "dtypes", "stride", "positions", "plan", "fanout"],
                    help="print one of the tables instead of the JSON line")
    ap.add_argument("--min", type=int, default=1 << 10, help="sweep tables: smallest size")
    ap.add_argument("--max", type=int, default=1 << 30, help="sweep tables: largest size")
    ap.add_argument("--k", type=int, nargs="+", default=[8, 4, 2], help="dtypes / stride / positions tables: inputs")
    ap.add_argument("--mib", type=int, default=256, help="dtypes / stride / positions tables: MiB per input")
    ap.add_argument("--sets", type=int, default=2, help="dtypes / stride / positions tables: buffer sets used in turn")
    ap.add_argument("--once", action="store_true", help="positions table: one launch per case, no timing")
    ap.add_argument("--loads", type=int, default=-1,
                    help="stride table: inputs in flight per wavefront for the cap columns (-1: the library's choice)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        log("bench.py: this build runs on ONE GPU (the k ranks are k HBM buffers on it); "
            "--gpus %d is not supported" % args.gpus)
        sys.exit(2)

    import torch
    from flagcx_amd import local as L
    if not torch.cuda.is_available():
        log("bench.py: no GPU visible")
        sys.exit(1)
    torch.cuda.set_device(0)
    L.check(L.lib().flagcxLocalInit())

    if args.table:
        {"sweep": table_sweep, "sweep-rotate": table_sweep, "configs": table_configs, "dtypes": table_dtypes,
         "stride": table_stride, "positions": table_positions, "plan": table_plan, "fanout": table_fanout}[args.table](L, args)
        return

    # The 8 input buffers and the output live in one allocation, at the addresses
    # flagcxLocalPlaceBuffers gives: equal offsets into them fall into different HBM
    # channel groups, which is how a caller that owns the ranks' staging buffers would
    # lay them out.  --allocator-layout takes nine separate torch allocations instead
    # (258 MiB apart on this allocator: all in one channel group).
    nbytes = N_ELEM * 2
    bufs, pool = placed(L, K + 1, N_ELEM, torch.bfloat16, args.allocator_layout)
    layout = "nine separate torch allocations" if args.allocator_layout else \
        "one allocation, buffers placed by flagcxLocalPlaceBuffers"
    # seeded synthetic inputs: N(0,1) per input from seeds 0..7, rounded to bf16
    inputs = bufs[:K]
    out = bufs[K]
    for seed in range(K):
        g = torch.Generator(device="cuda").manual_seed(seed)
        inputs[seed].copy_(torch.randn(N_ELEM, generator=g, device="cuda", dtype=torch.float32))
    torch.cuda.synchronize()

    def step():
        L.reduce(inputs, out, L.RedOp.Sum)

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()                      # same stream the launches go to
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / args.steps
    kern_ms = ev0.elapsed_time(ev1) / args.steps
    value = ALGO_BYTES / (wall_ms * 1e-3) / 1e9
    achieved = ALGO_BYTES / (kern_ms * 1e-3) / 1e9

    # The timed loop above reduces the same nine buffers every step, as the metric is
    # defined; part of the 256 MiB output of one step is then still in the memory-side
    # cache when the next step writes it again.  For comparison: S sets of buffers
    # used in turn, so that no launch finds anything of its own there.
    rotating = None
    if args.rotate_sets >= 2:
        sets, keep = [bufs], []
        for _ in range(args.rotate_sets - 1):
            more, p2 = placed(L, K + 1, N_ELEM, torch.bfloat16, args.allocator_layout)
            keep.append(p2)
            for j in range(K):
                more[j].copy_(inputs[j])
            sets.append(more)
        nset = len(sets)
        rot_ms = timed_sets_ms(lambda i: L.reduce(sets[i][:K], sets[i][K], L.RedOp.Sum), nset,
                               warmup=2 * nset, iters=args.steps)
        same_out = all(torch.equal(sets[i][K].view(torch.int16), out.view(torch.int16)) for i in range(1, nset))
        rotating = {"sets": nset, "value": round(ALGO_BYTES / (rot_ms * 1e-3) / 1e9, 1), "unit": "GB/s",
                    "frac": round(ALGO_BYTES / (rot_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
                    "avg_launch_ms": round(rot_ms, 5), "outputs_equal_first_set": bool(same_out)}
        del sets, keep
        torch.cuda.empty_cache()

    for _ in range(args.calibrate_copy):
        L.memcpy(out.data_ptr(), inputs[0].data_ptr(), N_ELEM * 2)
    torch.cuda.synchronize()

    # small-message latency: 2-input fp32 sum over 4 KiB buffers, arguments
    # marshalled once so the loop is one C call per launch
    a = torch.rand(1024, device="cuda")
    b = torch.rand(1024, device="cuda")
    c = torch.empty(1024, device="cuda")
    ptrs = (C.c_void_p * 2)(a.data_ptr(), b.data_ptr())
    st = L.current_stream()
    sref = C.byref(st)
    fn = L.lib().flagcxLocalReduce
    cptr, f32, opsum = c.data_ptr(), int(L.DataType.Float32), int(L.RedOp.Sum)

    def small():
        return fn(ptrs, 2, cptr, 1024, f32, opsum, sref)

    lat_stream_us = timed_ms(small, warmup=200, iters=2000) * 1e3
    singles = []
    for _ in range(200):
        s0 = time.perf_counter()
        small()
        torch.cuda.synchronize()
        singles.append((time.perf_counter() - s0) * 1e6)
    singles.sort()

    # what the GPU itself takes per launch: 1000 of them captured once into a HIP graph and replayed
    graph_us = None
    try:
        side = torch.cuda.Stream()
        sst = L.Stream(side.cuda_stream)
        ssref = C.byref(sst)
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(10):
                fn(ptrs, 2, cptr, 1024, f32, opsum, ssref)
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            for _ in range(1000):
                fn(ptrs, 2, cptr, 1024, f32, opsum, ssref)
        graph_us = timed_ms(graph.replay, warmup=3, iters=5)
        del graph
    except Exception as e:
        log("bench.py: graph replay of small launches failed: %r" % (e,))

    # the same figure as a C caller sees it (no interpreter in the launch path), beside the runtime's
    # own floor: an empty kernel and a 4 KiB hipMemcpyAsync timed the same way
    c_lat = None
    floor = latency_floor()
    if floor and "library_reduce2_fp32" in floor:
        c_lat = {"back_to_back_per_launch": floor["library_reduce2_fp32"]["back_to_back"],
                 "single_launch_to_sync_median": floor["library_reduce2_fp32"]["launch_to_sync"]}

    result = {
        "metric": "hbm_gbps_reduce8_bf16_sum_256MiB", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": "8-input bf16 sum reduce, fp32 accumulation, 256 MiB per input buffer "
                               "(128Mi elements), N(0,1) from seeds 0..7",
                   "nranks": K, "elements": N_ELEM, "bytes_per_step": ALGO_BYTES, "accumulate": "fp32",
                   "buffers": layout},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "rotating_buffers": rotating,
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": TRAFFIC_BYTES,
                     "traffic_source": TRAFFIC_SOURCE + " (rocprofv3 counter runs of this same command, "
                                                        "not measured by this run)",
                     "kernel": "reduceWaveKernel<bf16,sum,K=8,U=1,TILED=false>", "avg_launch_ms": round(kern_ms, 5),
                     "algorithmic_bytes_per_launch": ALGO_BYTES},
        "latency_us_4KiB": {"workload": "2-input fp32 sum, 4 KiB per buffer",
                            "c_caller": c_lat,
                            "c_caller_beside_the_runtime_floor": floor,
                            "hip_graph_replay_per_launch": None if graph_us is None else round(graph_us, 3),
                            "note": "back to back from a caller, every launch costs what the runtime takes on the host "
                                    "to launch ANY kernel with arguments (minimal_sum_kernel_4x64, hipMemcpyAsync_d2d); "
                                    "the GPU itself takes such launches as fast as empty ones (hip_graph_replay_per_launch)",
                            "python_ctypes_caller": {
                                "back_to_back_per_launch": round(lat_stream_us, 3),
                                "single_launch_to_sync_median": round(singles[len(singles) // 2], 3)}},
    }

    if not args.no_cpu:
        bits = [t.view(torch.int16) for t in inputs]
        sample = min(args.cpu_sample, N_ELEM)
        base, host, dst = cpu_headline(bits, sample)
        result["cpu_baseline"] = base
        # spot check of the GPU result against the oracle on the sample
        got = out[:sample].view(torch.int16).cpu().numpy().view(np.uint16)
        result["spot_check_vs_oracle"] = "bit-exact" if got.tobytes() == dst.tobytes() else "MISMATCH"
        if result["spot_check_vs_oracle"] != "bit-exact":
            log("bench.py: GPU result differs from the oracle on the sample")
            print(json.dumps(result))
            sys.exit(1)
        del host, dst

    variants = None
    if not args.no_configs:
        variants = config_headline_variants(L, inputs)
    del bufs, pool, inputs, out
    torch.cuda.empty_cache()

    # what the memory system of THIS box gives (a child process of its own, nothing else on the GPU meanwhile)
    ceiling = measured_ceiling()
    if ceiling:
        result["roofline"]["ceiling"] = ceiling
        if ceiling.get("best_read_only"):
            result["roofline"]["frac_of_best_read_only"] = round(achieved / ceiling["best_read_only"], 4)

    if not args.no_configs:
        cfg = {"method": "5 warm-up + 20 timed back-to-back passes per row, HIP events on the launch stream; "
                         "C5 rows: median of 20 single launches, each between its own event pair; "
                         "frac = GB/s / 8000; buffers placed by flagcxLocalPlaceBuffers unless "
                         "--allocator-layout"}
        # the rows below are additions to the line: whatever goes wrong in one of them is reported in its
        # place, and the headline figures above are printed all the same
        try:
            c1_rows, (ca, cb, cout) = config_c1(L, args.allocator_layout)
            cfg.update(c1_rows)
            if not args.no_cpu:
                c1_cpu, ha, hb = cpu_c1_reference_path()
                result["cpu_baseline"]["c1_fp32_reference_path"] = c1_cpu
                # the GPU's C1 output against the same sum on the host (fp32 add is exact either way)
                L.reduce([ca, cb], cout, L.RedOp.Sum)
                torch.cuda.synchronize()
                ga, gb = ca.cpu().numpy(), cb.cpu().numpy()
                cfg["C1_same_buffers"]["bit_exact_vs_host_sum"] = bool(np.array_equal(cout.cpu().numpy(), ga + gb))
                del ha, hb
            del ca, cb, cout
            torch.cuda.empty_cache()
        except Exception as e:
            cfg["C1_error"] = repr(e)
            log("bench.py: configuration C1 failed: %r" % (e,))
        cfg.update(variants or {})
        for name, fn in (("C3", lambda: config_c3(L, full=False, separate=args.allocator_layout)),
                         ("C4", lambda: config_c4(L, args.allocator_layout)), ("C5", lambda: config_c5(L)),
                         ("fanout", lambda: config_fanout(L)), ("plan", lambda: config_plan_replay(L))):
            try:
                cfg.update(fn())
            except Exception as e:
                cfg[name + "_error"] = repr(e)
                log("bench.py: configuration %s failed: %r" % (name, e))
        result["configs"] = cfg

    print(json.dumps(result))


if __name__ == "__main__":
    main()
