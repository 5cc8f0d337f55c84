"""GPU tests of the host-producer / device-consumer reduce queue (flagcxLocalReduceFifo*),
through the C ABI, against the CPU oracle.  Same bar as the launch-per-call reduce:
bit equality with the oracle; where an arithmetic result is NaN any payload passes.

Every test bounds the consumer's idle limit first, so a mistake ends in a timed-out
queue and a failed assertion, not in a resident kernel that waits for minutes.
"""
import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import DT_NAME, OP_NAME, dev_empty, from_dev, is_float, make_inputs, same, to_dev

pytestmark = pytest.mark.gpu

RUNNING, STOPPED, TIMED_OUT, PARKED = 1, 2, 3, 4
ALIVE = (RUNNING, PARKED)


@pytest.fixture(scope="module")
def L():
    import torch
    assert torch.cuda.is_available()
    from flagcx_amd import local
    assert local.lib().flagcxLocalInit() == 0
    local.lib().flagcxLocalSetMaxSpinCount(1 << 19)
    yield local
    local.lib().flagcxLocalSetMaxSpinCount(-1)


def nan_ok(dtype, op):
    return is_float(dtype) and op in (O.SUM, O.PROD, O.AVG)


def expect(srcs, dt, op):
    rc, want = O.reduce([np.ascontiguousarray(s) for s in srcs], dt, op)
    assert rc == 0
    return want


CASES = [
    (O.BF16, O.SUM, 8), (O.FP16, O.AVG, 8), (O.FP32, O.SUM, 2), (O.INT32, O.MAX, 4), (O.INT32, O.MIN, 4),
    (O.FP64, O.PROD, 3), (O.INT8, O.MIN, 5), (O.UINT8, O.SUM, 7), (O.INT64, O.SUM, 6), (O.BF16, O.MAX, 8),
    (O.FP16, O.MIN, 2), (O.UINT64, O.MAX, 1), (O.FP32, O.AVG, 3), (O.UINT32, O.PROD, 2),
]


@pytest.mark.parametrize("dt,op,k", CASES, ids=lambda v: str(v))
def test_fifo_reduce_matches_oracle(L, dt, op, k):
    """Several entries of different, ragged sizes in one run of the consumer."""
    import torch
    counts = [1, 7, 1023, 4097, (1 << 18) + 3, 64 * 1024]
    ins = [make_inputs(dt, k, n, seed=100 + i, op=op) for i, n in enumerate(counts)]
    devs = [[to_dev(a) for a in group] for group in ins]
    outs = [dev_empty(n, ins[0][0].dtype.itemsize, fill=0x55) for n in counts]
    torch.cuda.synchronize()
    q = L.ReduceFifo(16, k, dt, op)
    try:
        with q:
            assert q.grid() >= 2
            tickets = [q.enqueue_reduce([d.data_ptr() for d in devs[i]], outs[i].data_ptr(), counts[i])
                       for i in range(len(counts))]
            assert tickets == list(range(1, len(counts) + 1))
            q.wait(tickets[-1])
            assert q.query()[:2] == (len(counts), len(counts))
        assert q.query()[2] == STOPPED
    finally:
        q.close()
    for i, n in enumerate(counts):
        got = from_dev(outs[i], ins[i][0].dtype)
        assert same(got, expect(ins[i], dt, op), nan_class=nan_ok(dt, op), dtype=dt), (DT_NAME[dt], OP_NAME[op], n)


@pytest.mark.parametrize("dt,op,k", [(O.BF16, O.SUM, 8), (O.FP32, O.SUM, 3), (O.INT8, O.MAX, 4), (O.FP64, O.MIN, 2)],
                         ids=lambda v: str(v))
def test_fifo_misaligned_and_in_place(L, dt, op, k):
    """Element-aligned pointers: a shared offset (head/tail peel), sources at other
    offsets modulo 16 (unaligned loads), and recvbuff == sendbuffs[0]."""
    import torch
    n = 50_000
    isz = np.dtype(O.NP_OF[dt]).itemsize
    pad = 16 // isz
    ins = make_inputs(dt, k, n + 8 * pad, seed=7, op=op)
    devs = [to_dev(a) for a in ins]
    out_a = dev_empty(n + 2 * pad, isz, fill=0)
    out_d = dev_empty(n + 8 * pad, isz, fill=0)
    out_b = dev_empty(n + 2 * pad, isz, fill=0)
    torch.cuda.synchronize()
    # a: every pointer shifted by one element; b: source j shifted by j % pad elements, dst by 1
    offs_b = [(j + 2) % pad if pad > 1 else 0 for j in range(k)]
    inplace = devs[0].clone()
    torch.cuda.synchronize()
    q = L.ReduceFifo(8, k, dt, op)
    try:
        with q:
            q.enqueue_reduce([d.data_ptr() + isz for d in devs], out_a.data_ptr() + isz, n)
            q.enqueue_reduce([d.data_ptr() + offs_b[j] * isz for j, d in enumerate(devs)], out_b.data_ptr() + isz, n)
            q.enqueue_reduce([inplace.data_ptr()] + [d.data_ptr() for d in devs[1:]], inplace.data_ptr(), n)
            # d: 16-byte aligned, 80 bytes into a cache line (sources) and 48 bytes (destination): short first unit
            q.enqueue_reduce([d.data_ptr() + 80 for d in devs], out_d.data_ptr() + 48, n)
    finally:
        q.close()
    npdt = ins[0].dtype
    got_a = from_dev(out_a, npdt)
    assert same(got_a[1:n + 1], expect([a[1:n + 1] for a in ins], dt, op), nan_class=nan_ok(dt, op), dtype=dt)
    assert not got_a[0].tobytes().strip(b"\0") and not got_a[n + 1:].tobytes().strip(b"\0")  # guards untouched
    got_b = from_dev(out_b, npdt)
    want_b = expect([a[offs_b[j]:offs_b[j] + n] for j, a in enumerate(ins)], dt, op)
    assert same(got_b[1:n + 1], want_b, nan_class=nan_ok(dt, op), dtype=dt)
    assert not got_b[0].tobytes().strip(b"\0") and not got_b[n + 1:].tobytes().strip(b"\0")
    got_d = from_dev(out_d, npdt)
    so, do = 80 // isz, 48 // isz
    assert same(got_d[do:do + n], expect([a[so:so + n] for a in ins], dt, op), nan_class=nan_ok(dt, op), dtype=dt)
    assert not got_d[:do].tobytes().strip(b"\0") and not got_d[do + n:].tobytes().strip(b"\0")
    got_c = from_dev(inplace, npdt)
    assert same(got_c[:n], expect([a[:n] for a in ins], dt, op), nan_class=nan_ok(dt, op), dtype=dt)
    assert same(got_c[n:n + 2 * pad], ins[0][n:n + 2 * pad])


def test_fifo_triggers_chain(L):
    """Binary triggers in the reference's 256-bit layout: addr3 = OP(addr1, addr2).
    A k-way sum as a chain through one accumulator."""
    import torch
    dt, op, k, n = O.FP32, O.SUM, 5, 300_001
    ins = make_inputs(dt, k, n, seed=11)
    devs = [to_dev(a) for a in ins]
    acc = dev_empty(n, 4, fill=0)
    torch.cuda.synchronize()
    q = L.ReduceFifo(4, 2, dt, op)
    try:
        with q:
            # acc = in1 + in0, then acc = in_j + acc
            # (no waits in between: the queue itself orders an entry behind the one it depends on)
            t = q.enqueue(L.ReduceTrigger.make(devs[1].data_ptr(), devs[0].data_ptr(), acc.data_ptr(), n, dt, op))
            for j in range(2, k):
                t = q.enqueue(L.ReduceTrigger.make(devs[j].data_ptr(), acc.data_ptr(), acc.data_ptr(), n, dt, op))
            q.wait(t)
            # results are visible to a host copy while the consumer is still resident
            got_live = from_dev(acc, np.float32)
            bad = L.ReduceTrigger.make(devs[0].data_ptr(), devs[1].data_ptr(), acc.data_ptr(), n, O.FP64, op)
            with pytest.raises(L.FlagcxError):
                q.enqueue(bad)
    finally:
        q.close()
    want = expect(ins, dt, op)
    assert same(got_live, want, nan_class=True, dtype=dt)
    assert same(from_dev(acc, np.float32), want, nan_class=True, dtype=dt)


def test_fifo_sees_inputs_rewritten_while_resident(L):
    """The same small buffers (they would stay in cache) are rewritten between entries,
    by a host-to-device copy and by a copy kernel on another stream, while the consumer
    stays resident: every entry must fold the new contents, and its result must be
    what a host copy and another stream's kernel read afterwards."""
    import torch
    dt, op, k, n = O.INT32, O.SUM, 4, 16 * 1024
    rounds = 12
    rng = np.random.default_rng(3)
    host = [[rng.integers(-2**31, 2**31 - 1, n, dtype=np.int32) for _ in range(k)] for _ in range(rounds)]
    staged = [[torch.from_numpy(a).cuda() for a in group] for group in host]   # sources of the copy kernel
    pinned = [[torch.from_numpy(a).pin_memory() for a in group] for group in host]
    devs = [torch.zeros(n, dtype=torch.int32, device="cuda") for _ in range(k)]
    out = torch.zeros(n, dtype=torch.int32, device="cuda")
    echo = torch.zeros(n, dtype=torch.int32, device="cuda")
    side = torch.cuda.Stream()
    side_ref = L.Stream(side.cuda_stream)
    torch.cuda.synchronize()
    got_host, got_echo = [], []
    q = L.ReduceFifo(8, k, dt, op)
    try:
        with q:
            for r in range(rounds):
                for j in range(k):
                    if r % 2 == 0:
                        with torch.cuda.stream(side):
                            devs[j].copy_(pinned[r][j], non_blocking=True)      # copy engine
                    else:
                        L.memcpy(devs[j].data_ptr(), staged[r][j].data_ptr(), n * 4, stream=side_ref)  # kernel
                side.synchronize()
                q.wait(q.enqueue_reduce([d.data_ptr() for d in devs], out.data_ptr(), n))
                L.memcpy(echo.data_ptr(), out.data_ptr(), n * 4, stream=side_ref)
                side.synchronize()
                got_echo.append(echo.cpu().numpy().copy())
                got_host.append(out.cpu().numpy().copy())
    finally:
        q.close()
    for r in range(rounds):
        want = expect(host[r], dt, op)
        assert same(got_host[r], want), r
        assert same(got_echo[r], want), r


def test_other_launches_run_next_to_the_resident_consumer(L):
    """An ordinary 8-input reduce (which reserves LDS) and a copy on another stream
    finish while the consumer stays resident and keeps serving entries."""
    import torch
    dt, op, k, n = O.BF16, O.SUM, 8, 1 << 20
    ins = make_inputs(dt, k, n, seed=21)
    devs = [to_dev(a) for a in ins]
    out_q = dev_empty(n, 2, fill=0)
    out_l = dev_empty(n, 2, fill=0)
    out_c = dev_empty(n, 2, fill=0)
    side = torch.cuda.Stream()
    st = L.Stream(side.cuda_stream)
    torch.cuda.synchronize()
    q = L.ReduceFifo(8, k, dt, op)
    try:
        with q:
            L.reduce(devs, out_l, op, dtype=dt, stream=st)
            L.memcpy(out_c.data_ptr(), out_l.data_ptr(), n * 2, stream=st)
            side.synchronize()
            assert q.query()[2] in ALIVE
            q.wait(q.enqueue_reduce([d.data_ptr() for d in devs], out_q.data_ptr(), n))
            assert q.query()[2] in ALIVE
    finally:
        q.close()
    want = expect(ins, dt, op)
    for got in (out_q, out_l, out_c):
        assert same(from_dev(got, np.uint16), want, nan_class=True, dtype=dt)


def test_fifo_orders_dependent_entries(L):
    """Entries are folded concurrently unless one touches what another still in flight
    reads or writes; then the result must be that of running them one after another.
    Read-after-write, write-after-read and write-after-write, between independent ones."""
    import torch
    dt, op, n = O.INT32, O.SUM, 1_500_001
    rng = np.random.default_rng(9)
    h = {name: rng.integers(-2**31, 2**31 - 1, n, dtype=np.int32) for name in "abcdefg"}
    d = {name: to_dev(v) for name, v in h.items()}
    outs = {name: dev_empty(n, 4, fill=0) for name in ("p", "q", "r", "s")}
    torch.cuda.synchronize()
    P = lambda name: (d[name] if name in d else outs[name]).data_ptr()
    program = [                      # (dst, srcs)
        ("p", ["a", "b"]),           # p = a + b
        ("a", ["c", "d"]),           # overwrites a while p may still be reading it
        ("q", ["p", "a", "e"]),      # reads both results
        ("r", ["f", "g"]),           # independent
        ("q", ["q", "r"]),           # in place on q, needs q and r
        ("s", ["e", "f"]),           # independent
        ("s", ["g", "g"]),           # overwrites s
    ]
    q = L.ReduceFifo(4, 3, dt, op)
    try:
        with q:
            for _ in range(3):       # several times over, through a ring of 4 slots
                for dst, srcs in program:
                    t = q.enqueue_reduce([P(x) for x in srcs], P(dst), n)
            q.wait(t)
    finally:
        q.close()
    env = {k_: v.copy() for k_, v in h.items()}
    for _ in range(3):
        for dst, srcs in program:
            env[dst] = expect([env[x] for x in srcs], dt, op)
    for name in ("p", "q", "r", "s"):
        assert same(from_dev(outs[name], np.int32), env[name]), name
    assert same(from_dev(d["a"], np.int32), env["a"])


def test_fifo_several_producer_threads(L):
    """Four host threads append to one queue at once (a one-slot-per-thread ring, so they
    also meet 'full'); every entry is folded exactly once into its own output."""
    import threading
    import torch
    dt, op, k, n = O.FP32, O.SUM, 2, 40_003
    nthreads, per = 4, 25
    ins = [make_inputs(dt, k, n, seed=500 + t) for t in range(nthreads)]
    devs = [[to_dev(a) for a in g] for g in ins]
    outs = [[dev_empty(n, 4, fill=0) for _ in range(per)] for _ in range(nthreads)]
    torch.cuda.synchronize()
    errors, last = [], [0] * nthreads
    q = L.ReduceFifo(4, k, dt, op)
    try:
        with q:
            def produce(t):
                try:
                    for i in range(per):
                        last[t] = q.enqueue_reduce([d.data_ptr() for d in devs[t]], outs[t][i].data_ptr(), n)
                except Exception as e:
                    errors.append(repr(e))
            threads = [threading.Thread(target=produce, args=(t,)) for t in range(nthreads)]
            for th in threads:
                th.start()
            for th in threads:
                th.join(60)
            assert not errors, errors
            q.wait(max(last))
            assert q.query()[:2] == (nthreads * per, nthreads * per)
    finally:
        q.close()
    for t in range(nthreads):
        want = expect(ins[t], dt, op)
        for i in range(per):
            assert same(from_dev(outs[t][i], np.float32), want, nan_class=True, dtype=dt), (t, i)


def test_fifo_ring_wraps_and_restarts(L):
    """More entries than slots (the producer sees 'full' and retries), then a second
    start on the same queue with counters back at zero."""
    import torch
    dt, op, k, n = O.INT32, O.SUM, 3, 70_001
    rounds = 37
    ins = [make_inputs(dt, k, n, seed=300 + r) for r in range(4)]
    devs = [[to_dev(a) for a in g] for g in ins]
    outs = [dev_empty(n, 4, fill=0) for _ in range(rounds)]
    torch.cuda.synchronize()
    q = L.ReduceFifo(4, k, dt, op)
    try:
        for attempt in range(2):
            with q:
                full_seen = 0
                for r in range(rounds):
                    while True:
                        t = q.try_enqueue_reduce([d.data_ptr() for d in devs[r % 4]], outs[r].data_ptr(), n)
                        if t is not None:
                            break
                        full_seen += 1
                    assert t == r + 1
                    p, c, st = q.query()
                    assert p - c <= 4 and st in ALIVE
            p, c, st = q.query()
            assert (p, c, st) == (rounds + 1, rounds + 1, STOPPED)  # + the stop entry
            for r in range(rounds):
                assert same(from_dev(outs[r], np.int32), expect(ins[r % 4], dt, op)), (attempt, r)
                outs[r].zero_()
            torch.cuda.synchronize()
    finally:
        q.close()


def test_fifo_consumer_gives_up_when_idle(L):
    """With parking switched off and a tiny spin limit, a consumer that never gets an
    entry leaves by itself, the queue reports it, and a restart works.  Every
    wavefront exits normally."""
    import time
    import torch
    dt, op = O.FP32, O.SUM
    ins = make_inputs(dt, 2, 5000, seed=5)
    devs = [to_dev(a) for a in ins]
    out = dev_empty(5000, 4, fill=0)
    torch.cuda.synchronize()
    L.lib().flagcxLocalSetMaxSpinCount(2000)
    q = L.ReduceFifo(4, 2, dt, op)
    q.set_linger(0)
    try:
        q.start()
        deadline = time.time() + 60
        while q.query()[2] == RUNNING and time.time() < deadline:
            time.sleep(0.01)
        assert q.query()[2] == TIMED_OUT
        with pytest.raises(L.FlagcxError):
            q.enqueue_reduce([d.data_ptr() for d in devs], out.data_ptr(), 5000)
        with pytest.raises(L.FlagcxError):
            q.stop()
        L.lib().flagcxLocalSetMaxSpinCount(1 << 19)
        with q:
            q.enqueue_reduce([d.data_ptr() for d in devs], out.data_ptr(), 5000)
        assert same(from_dev(out, np.float32), expect(ins, dt, op), nan_class=True, dtype=dt)
    finally:
        L.lib().flagcxLocalSetMaxSpinCount(1 << 19)
        q.close()


def test_fifo_parks_when_idle_and_comes_back(L):
    """Nothing outstanding for `linger` polls: the kernel ends (a device-wide
    synchronisation returns), the queue stays usable, and the next entry launches the
    consumer again with the counters carried on.  Several idle gaps, a stop while
    parked, and a restart."""
    import time
    import torch
    dt, op, k, n = O.BF16, O.SUM, 8, 300_000
    ins = [make_inputs(dt, k, n, seed=60 + r) for r in range(3)]
    devs = [[to_dev(a) for a in g] for g in ins]
    outs = [dev_empty(n, 2, fill=0) for _ in range(6)]
    torch.cuda.synchronize()
    q = L.ReduceFifo(4, k, dt, op)
    q.set_linger(16)
    try:
        q.start()
        tickets = []
        for r in range(6):
            tickets.append(q.enqueue_reduce([d.data_ptr() for d in devs[r % 3]], outs[r].data_ptr(), n))
            q.wait(tickets[-1])
            if r % 2 == 1:
                deadline = time.time() + 30
                while q.query()[2] != PARKED and time.time() < deadline:
                    time.sleep(0.001)
                assert q.query()[2] == PARKED
                torch.cuda.synchronize()          # returns: no kernel is left on the GPU
                p, c, _ = q.query()
                assert p == c == r + 1
        assert tickets == [1, 2, 3, 4, 5, 6]
        q.stop()                                  # parked at this point
        assert q.query() == (7, 7, STOPPED)
        for r in range(6):
            assert same(from_dev(outs[r], np.uint16), expect(ins[r % 3], dt, op), nan_class=True, dtype=dt), r
            outs[r].zero_()
        torch.cuda.synchronize()
        with q:                                   # counters start again at zero
            assert q.enqueue_reduce([d.data_ptr() for d in devs[0]], outs[0].data_ptr(), n) == 1
        assert same(from_dev(outs[0], np.uint16), expect(ins[0], dt, op), nan_class=True, dtype=dt)
    finally:
        q.close()


def test_fifo_chunked_shard_matches_single_launch(L):
    """A reduce-scatter shard cut into 4 MiB chunks and fed chunk by chunk gives the
    bytes of one launch over the whole shard (fp16 avg, 8 inputs)."""
    import torch
    dt, op, k = O.FP16, O.AVG, 8
    chunk = 2 * 1024 * 1024  # elements = 4 MiB
    nchunks = 8
    n = chunk * nchunks
    g = torch.Generator(device="cuda").manual_seed(1)
    devs = [(torch.randn(n, generator=g, device="cuda") * 0.01).to(torch.float16) for _ in range(k)]
    whole = torch.empty(n, dtype=torch.float16, device="cuda")
    piecewise = torch.zeros(n, dtype=torch.float16, device="cuda")
    L.reduce(devs, whole, op, dtype=dt)
    torch.cuda.synchronize()
    q = L.ReduceFifo(16, k, dt, op)
    try:
        with q:
            for c in range(nchunks):
                q.enqueue_reduce([d.data_ptr() + c * chunk * 2 for d in devs], piecewise.data_ptr() + c * chunk * 2,
                                 chunk)
    finally:
        q.close()
    assert torch.equal(whole.view(torch.int16), piecewise.view(torch.int16))
    sample = slice(0, 4096)
    want = expect([d[sample].view(torch.int16).cpu().numpy().view(np.float16) for d in devs], dt, op)
    assert same(piecewise[sample].view(torch.int16).cpu().numpy().view(np.float16), want, nan_class=True, dtype=dt)


def test_consumer_on_a_queue_of_its_own_holds_no_stream_up(L):
    """With flagcxLocalReduceFifoSetOwnQueue no stream shares the consumer's hardware queue: launches on many
    other streams finish while a consumer that never parks sits on the GPU.  (Without it some of these
    streams would wait until the consumer leaves, here at its spin bound, seconds later.)"""
    import time
    import torch
    dt, op, n = O.FP32, O.SUM, 4096
    ins = make_inputs(dt, 2, n, seed=77, op=op)
    devs = [to_dev(a) for a in ins]
    out = dev_empty(n, 4, fill=0)
    others = [torch.cuda.Stream() for _ in range(12)]
    work = [torch.zeros(1024, dtype=torch.int32, device="cuda") for _ in others]
    torch.cuda.synchronize()
    q = L.ReduceFifo(8, 2, dt, op)
    try:
        q.set_linger(0)
        q.set_own_queue(True)
        with q:
            q.wait(q.enqueue_reduce([d.data_ptr() for d in devs], out.data_ptr(), n))
            t0 = time.perf_counter()
            for s, w in zip(others, work):
                with torch.cuda.stream(s):
                    w.add_(1)
                s.synchronize()
            elapsed = time.perf_counter() - t0
            assert q.query()[2] == RUNNING
        assert elapsed < 0.25, elapsed
    finally:
        q.close()
    assert all(int(w[0].item()) == 1 for w in work)
    assert same(from_dev(out, np.float32), expect(ins, dt, op), nan_class=True, dtype=dt)
    # switching back gives an ordinary stream again, and the queue still works
    q = L.ReduceFifo(8, 2, dt, op)
    try:
        q.set_own_queue(True)
        q.set_own_queue(False)
        out.zero_()
        torch.cuda.synchronize()
        with q:
            q.wait(q.enqueue_reduce([d.data_ptr() for d in devs], out.data_ptr(), n))
            with pytest.raises(L.FlagcxError) as e:
                q.set_own_queue(True)
            assert e.value.code == L.Result.InvalidUsage
    finally:
        q.close()
    assert same(from_dev(out, np.float32), expect(ins, dt, op), nan_class=True, dtype=dt)


def test_random_chains_of_dependent_entries_replay_in_order(L):
    """Seeded random runs of entries over a small pool of buffers: sources repeat, the destination may be one of
    the sources, later entries read and overwrite what earlier ones wrote, over sub-ranges.  The queue must give
    what running the entries one after another gives (replayed on the CPU through the oracle)."""
    import random
    import torch
    rnd = random.Random(4242)
    for case in range(160):
        dt, op = rnd.choice([(O.INT32, O.SUM), (O.FP32, O.SUM), (O.INT32, O.MAX), (O.FP32, O.PROD), (O.INT64, O.MIN)])
        npdt = np.dtype(O.NP_OF[dt])
        isz = npdt.itemsize
        nbuf, n = rnd.randint(3, 7), rnd.choice([64, 1000, 4096, rnd.randint(1, 100_000)])
        rng = np.random.default_rng(rnd.randint(0, 1 << 30))
        if npdt.kind == "f":
            host = [(1.0 + 0.01 * rng.standard_normal(n)).astype(npdt) for _ in range(nbuf)]
        else:
            host = [rng.integers(-1000, 1000, n).astype(npdt) for _ in range(nbuf)]
        dev = [to_dev(h) for h in host]
        torch.cuda.synchronize()
        maxk = rnd.randint(2, 8)
        q = L.ReduceFifo(rnd.choice([4, 8, 64]), maxk, dt, op)
        plan = []
        try:
            with q:
                ticket = 0
                for _ in range(rnd.randint(1, 40)):
                    srcs = [rnd.randrange(nbuf) for _ in range(rnd.randint(1, maxk))]
                    d = rnd.randrange(nbuf)
                    lo = rnd.randrange(0, n)
                    cnt = rnd.randint(1, n - lo)
                    plan.append((srcs, d, lo, cnt))
                    ticket = q.enqueue_reduce([dev[s].data_ptr() + lo * isz for s in srcs], dev[d].data_ptr() + lo * isz, cnt)
                q.wait(ticket)
        finally:
            q.close()
        torch.cuda.synchronize()
        for srcs, d, lo, cnt in plan:
            host[d][lo:lo + cnt] = expect([host[s][lo:lo + cnt] for s in srcs], dt, op)
        for i in range(nbuf):
            assert same(from_dev(dev[i], npdt), host[i], nan_class=True, dtype=dt), (case, dt, op, i, plan[:4])
