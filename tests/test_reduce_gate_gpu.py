"""GPU tests of the gated batch (flagcxLocalReduceBatchGated / flagcxLocalGate*), through the
C ABI, against the CPU oracle: a batch of reductions launched before its inputs are said to
be complete, folded as the host raises the gate's count.  Same bar as the launch-per-call
reduce: bit equality with the oracle; where an arithmetic result is NaN any payload passes.

Every test bounds the wait first, so a mistake ends in an abandoned launch and a failed
assertion, not in a kernel that waits for minutes.
"""
import time

import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import DT_NAME, OP_NAME, dev_empty, from_dev, is_float, make_inputs, same, to_dev

pytestmark = pytest.mark.gpu

OK, TIMED_OUT = 0, 1


@pytest.fixture(scope="module")
def L():
    import torch
    assert torch.cuda.is_available()
    from flagcx_amd import local
    assert local.lib().flagcxLocalInit() == 0
    local.lib().flagcxLocalSetMaxSpinCount(1 << 21)  # seconds: far above any pause of the host between two calls
    yield local
    local.lib().flagcxLocalSetMaxSpinCount(-1)


def nan_ok(dtype, op):
    return is_float(dtype) and op in (O.SUM, O.PROD, O.AVG)


def expect(srcs, dt, op):
    rc, want = O.reduce([np.ascontiguousarray(s) for s in srcs], dt, op)
    assert rc == 0
    return want


def untouched(t, fill=0x55):
    """Every element still holds what dev_empty(fill=...) put there."""
    return bool((t == fill).all().item())


CASES = [
    (O.BF16, O.SUM, 8), (O.FP16, O.AVG, 8), (O.FP32, O.SUM, 2), (O.INT32, O.MAX, 4), (O.FP64, O.PROD, 3),
    (O.INT8, O.MIN, 5), (O.UINT8, O.SUM, 7), (O.INT64, O.SUM, 6), (O.UINT64, O.MAX, 1), (O.UINT32, O.PROD, 2),
]


@pytest.mark.parametrize("dt,op,k", CASES, ids=lambda v: str(v))
def test_gated_batch_matches_oracle(L, dt, op, k):
    """Descriptors of different, ragged sizes; the count is raised in steps while the launch is on the GPU.
    (That a descriptor which is never opened is never written is what the give-up test below shows: work on
    another stream may be queued behind the waiting launch, so nothing is read while it waits.)"""
    import torch
    counts = [1, 7, 1023, 4097, (1 << 18) + 3, 64 * 1024]
    ins = [make_inputs(dt, k, n, seed=300 + i, op=op) for i, n in enumerate(counts)]
    isz = ins[0][0].dtype.itemsize
    devs = [[to_dev(a) for a in group] for group in ins]
    outs = [dev_empty(n, isz, fill=0x55) for n in counts]
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with L.Gate() as gate:
        with torch.cuda.stream(side):
            first = gate.reduce_batch([([d.data_ptr() for d in devs[i]], outs[i].data_ptr(), counts[i])
                                       for i in range(len(counts))], op, dt, k)
        assert first == 0
        assert gate.query() == (len(counts), 0, OK)
        for upto in (2, 3, 5, len(counts)):
            gate.open(upto)
            time.sleep(0.001)
        side.synchronize()
        assert gate.query() == (len(counts), len(counts), OK)
    for i, n in enumerate(counts):
        got = from_dev(outs[i], ins[i][0].dtype)
        assert same(got, expect(ins[i], dt, op), nan_class=nan_ok(dt, op), dtype=dt), (DT_NAME[dt], OP_NAME[op], n)


@pytest.mark.parametrize("dt,op,k", [(O.BF16, O.SUM, 8), (O.FP32, O.SUM, 3), (O.INT8, O.MAX, 4), (O.FP64, O.MIN, 2)],
                         ids=lambda v: str(v))
def test_gated_positions_and_in_place(L, dt, op, k):
    """A shared offset of one element (head and tail elements), buffers 80 and 48 bytes into a cache line
    (short first tile, runs of tiles per XCD), and recvbuff == sendbuffs[0]."""
    import torch
    n = 150_000
    isz = np.dtype(O.NP_OF[dt]).itemsize
    pad = 16 // isz
    ins = make_inputs(dt, k, n + 8 * pad, seed=17, op=op)
    devs = [to_dev(a) for a in ins]
    out_a = dev_empty(n + 2 * pad, isz, fill=0)
    out_d = dev_empty(n + 8 * pad, isz, fill=0)
    inplace = devs[0].clone()
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with L.Gate() as gate:
        with torch.cuda.stream(side):
            gate.reduce_batch([
                ([d.data_ptr() + isz for d in devs], out_a.data_ptr() + isz, n),
                ([inplace.data_ptr()] + [d.data_ptr() for d in devs[1:]], inplace.data_ptr(), n),
                ([d.data_ptr() + 80 for d in devs], out_d.data_ptr() + 48, n),
            ], op, dt, k)
        for upto in (1, 2, 3):
            time.sleep(0.001)
            gate.open(upto)
        side.synchronize()
        assert gate.query()[2] == OK
    npdt = ins[0].dtype
    got_a = from_dev(out_a, npdt)
    assert same(got_a[1:n + 1], expect([a[1:n + 1] for a in ins], dt, op), nan_class=nan_ok(dt, op), dtype=dt)
    assert not got_a[0].tobytes().strip(b"\0") and not got_a[n + 1:].tobytes().strip(b"\0")  # guards untouched
    got_d = from_dev(out_d, npdt)
    so, do = 80 // isz, 48 // isz
    assert same(got_d[do:do + n], expect([a[so:so + n] for a in ins], dt, op), nan_class=nan_ok(dt, op), dtype=dt)
    assert not got_d[:do].tobytes().strip(b"\0") and not got_d[do + n:].tobytes().strip(b"\0")
    got_c = from_dev(inplace, npdt)
    assert same(got_c[:n], expect([a[:n] for a in ins], dt, op), nan_class=nan_ok(dt, op), dtype=dt)
    assert same(got_c[n:n + 2 * pad], ins[0][n:n + 2 * pad])


def test_gated_more_descriptors_than_one_launch_and_numbering(L):
    """70 descriptors (three launches), some of them empty, then a second call on the same gate whose
    descriptors were opened before it was made."""
    import torch
    dt, op, k = O.FP32, O.SUM, 3
    counts = [(37 * i) % 5000 + (0 if i % 9 == 4 else 1) for i in range(70)]
    counts = [0 if i % 9 == 4 else c for i, c in enumerate(counts)]
    ins = [make_inputs(dt, k, max(n, 1), seed=500 + i, op=op) for i, n in enumerate(counts)]
    devs = [[to_dev(a) for a in group] for group in ins]
    outs = [dev_empty(max(n, 1), 4, fill=0x55) for n in counts]
    more = make_inputs(dt, k, 100_003, seed=999, op=op)
    more_dev = [to_dev(a) for a in more]
    more_out = dev_empty(100_003, 4, fill=0x55)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with L.Gate() as gate:
        with torch.cuda.stream(side):
            first = gate.reduce_batch([([d.data_ptr() for d in devs[i]], outs[i].data_ptr(), counts[i])
                                       for i in range(70)], op, dt, k)
        assert first == 0
        for upto in (10, 33, 34, 64, 69, 71):  # 71: the next call's descriptor as well
            gate.open(upto)
            time.sleep(0.001)
        gate.open(5)  # lower counts change nothing
        side.synchronize()
        assert gate.query() == (70, 71, OK)
        with torch.cuda.stream(side):
            assert gate.reduce_batch([([d.data_ptr() for d in more_dev], more_out.data_ptr(), 100_003)], op, dt, k) == 70
        side.synchronize()
        assert gate.query() == (71, 71, OK)
    for i, n in enumerate(counts):
        if n == 0:
            assert untouched(outs[i])
            continue
        assert same(from_dev(outs[i], np.float32)[:n], expect([a[:n] for a in ins[i]], dt, op), nan_class=True, dtype=dt), i
    assert same(from_dev(more_out, np.float32), expect(more, dt, op), nan_class=True, dtype=dt)


def test_gated_launch_gives_up_when_nothing_opens(L):
    """The host never raises the count: after the bounded number of polls every wavefront leaves,
    nothing has been written, the gate says so and takes no further launch."""
    import torch
    dt, op, k, n = O.BF16, O.SUM, 4, 1 << 20
    ins = make_inputs(dt, k, n, seed=3, op=op)
    devs = [to_dev(a) for a in ins]
    outs = [dev_empty(n, 2, fill=0x55) for _ in range(3)]
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    L.lib().flagcxLocalSetMaxSpinCount(2000)
    try:
        gate = L.Gate()
        gate.open(1)  # the first descriptor may run (opened before the launch, so no host timing is involved), the others never arrive
        with torch.cuda.stream(side):
            gate.reduce_batch([([d.data_ptr() for d in devs], o.data_ptr(), n) for o in outs], op, dt, k)
        side.synchronize()
        assert gate.query() == (3, 1, TIMED_OUT)
        assert same(from_dev(outs[0], ins[0].dtype), expect(ins, dt, op), nan_class=True, dtype=dt)
        assert untouched(outs[1]) and untouched(outs[2])
        with pytest.raises(L.FlagcxError) as e:
            gate.open(3)
        assert e.value.code == L.Result.InternalError
        with pytest.raises(L.FlagcxError) as e:
            with torch.cuda.stream(side):
                gate.reduce_batch([([d.data_ptr() for d in devs], outs[1].data_ptr(), n)], op, dt, k)
        assert e.value.code == L.Result.InternalError
        gate.destroy()
    finally:
        L.lib().flagcxLocalSetMaxSpinCount(1 << 21)


def test_gate_destroy_abandons_a_waiting_launch(L):
    import torch
    dt, op, k, n = O.INT32, O.SUM, 2, 1 << 18
    ins = make_inputs(dt, k, n, seed=5, op=op)
    devs = [to_dev(a) for a in ins]
    out = dev_empty(n, 4, fill=0x55)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    gate = L.Gate()
    with torch.cuda.stream(side):
        gate.reduce_batch([([d.data_ptr() for d in devs], out.data_ptr(), n)], op, dt, k)
    time.sleep(0.005)
    gate.destroy()
    side.synchronize()
    assert untouched(out)


def test_gated_batch_argument_errors(L):
    import torch
    dt, op = O.FP32, O.SUM
    a = [to_dev(np.zeros(1024, np.float32)) for _ in range(9)]
    out = dev_empty(1024, 4, fill=0)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    ptrs = [t.data_ptr() for t in a]
    with L.Gate() as gate:
        def bad(descs, k, stream="current"):
            with pytest.raises(L.FlagcxError) as e:
                with torch.cuda.stream(side):
                    gate.reduce_batch(descs, op, dt, k, stream=stream)
            assert e.value.code == L.Result.InvalidArgument
        bad([(ptrs[:2], out.data_ptr(), 16)], 2, stream=None)                      # blocking stream
        bad([(ptrs, out.data_ptr(), 16)], 9)                                       # more than 8 inputs
        bad([([ptrs[0] + 4, ptrs[1]], out.data_ptr(), 16)], 2)                     # sources differ modulo 16
        bad([(ptrs[:2], out.data_ptr(), 16), (ptrs[:2], out.data_ptr() + 32, 16)], 2)  # overlapping outputs
        bad([(ptrs[:2], 0, 16)], 2)                                                # NULL recvbuff
        # nothing of a refused call has been numbered or launched
        assert gate.query() == (0, 0, OK)
        with torch.cuda.stream(side):
            assert gate.reduce_batch([], op, dt, 2) == 0
        side.synchronize()


def test_c3_shard_streamed_through_the_gate(L):
    """8 ranks x 1 GiB fp16, N(0, sigma = 0.01); rank 3's 128 MiB shard as 32 descriptors of 4 MiB in ring
    order, launched up front and opened one by one: the same bytes as the one-launch reduce-scatter, and a
    window of them against the oracle."""
    import torch
    MiB = 1 << 20
    nranks, per_rank = 8, 512 * MiB
    shard = per_rank // nranks
    send = []
    for r in range(nranks):
        g = torch.Generator(device="cuda").manual_seed(100 + r)
        buf = torch.empty(per_rank, dtype=torch.float16, device="cuda")
        for s in range(nranks):
            buf[s * shard:(s + 1) * shard] = (torch.randn(shard, generator=g, device="cuda") * 0.01).to(torch.float16)
        send.append(buf)
    rank = 3
    fused = torch.empty(shard, dtype=torch.float16, device="cuda")
    gated = torch.zeros(shard, dtype=torch.float16, device="cuda")
    L.reduce_scatter(send, rank, fused, L.RedOp.Avg)
    chunk = L.CHUNKSIZE // 2
    descs = [([send[(rank + 1 + j) % nranks].data_ptr() + (rank * shard + c * chunk) * 2 for j in range(nranks)],
              gated.data_ptr() + c * chunk * 2, chunk) for c in range(shard // chunk)]
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with L.Gate() as gate:
        with torch.cuda.stream(side):
            first = gate.reduce_batch(descs, L.RedOp.Avg, L.DataType.Float16, nranks)
        for c in range(len(descs)):
            gate.open(first + c + 1)
        side.synchronize()
        assert gate.query() == (len(descs), len(descs), OK)
    equal = bool(torch.equal(fused.view(torch.int16), gated.view(torch.int16)))
    assert equal
    w0, w1 = 5 * MiB + 3, 6 * MiB + 3
    win = [send[(rank + 1 + j) % nranks][rank * shard + w0:rank * shard + w1].cpu().numpy() for j in range(nranks)]
    rc, want = O.reduce(win, O.FP16, O.AVG)
    assert rc == 0 and same(gated[w0:w1].cpu().numpy(), want)


def test_gate_opened_from_another_thread(L):
    """The proxy's shape: one thread launches and synchronises, another one raises the count as chunks complete."""
    import threading
    import torch
    dt, op, k, n, chunks = O.FP32, O.SUM, 4, 1 << 16, 48
    ins = make_inputs(dt, k, n * chunks, seed=21, op=op)
    devs = [to_dev(a) for a in ins]
    out = dev_empty(n * chunks, 4, fill=0x55)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with L.Gate() as gate:
        def proxy():
            for c in range(chunks):
                time.sleep(0.0002)
                gate.open(c + 1)
        t = threading.Thread(target=proxy)
        with torch.cuda.stream(side):
            gate.reduce_batch([([d.data_ptr() + c * n * 4 for d in devs], out.data_ptr() + c * n * 4, n)
                               for c in range(chunks)], op, dt, k)
        t.start()
        side.synchronize()
        t.join()
        assert gate.query() == (chunks, chunks, OK)
    assert same(from_dev(out, np.float32), expect(ins, dt, op), nan_class=True, dtype=dt)


def test_gate_with_its_count_in_ordinary_device_memory(L, monkeypatch):
    """The fallback for devices without uncached memory: vector reads of the count, same bytes."""
    import torch
    monkeypatch.setenv("FLAGCX_LOCAL_GATE_CACHED", "1")
    dt, op, k = O.BF16, O.SUM, 8
    counts = [5, 4097, (1 << 18) + 3, 1 << 20]
    ins = [make_inputs(dt, k, n, seed=700 + i, op=op) for i, n in enumerate(counts)]
    devs = [[to_dev(a) for a in group] for group in ins]
    outs = [dev_empty(n, 2, fill=0x55) for n in counts]
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    with L.Gate() as gate:
        with torch.cuda.stream(side):
            gate.reduce_batch([([d.data_ptr() for d in devs[i]], outs[i].data_ptr(), counts[i])
                               for i in range(len(counts))], op, dt, k)
        for upto in range(1, len(counts) + 1):
            time.sleep(0.001)
            gate.open(upto)
        side.synchronize()
        assert gate.query() == (len(counts), len(counts), OK)
    for i, n in enumerate(counts):
        assert same(from_dev(outs[i], ins[i][0].dtype), expect(ins[i], dt, op), nan_class=True, dtype=dt), n


def test_gated_launch_on_the_gates_own_stream_holds_nothing_up(L):
    """The pipeline the gate is for, in a process that holds many streams: each chunk's inputs are
    produced by copies on one of 12 other streams, then the chunk is opened.  On the gate's own stream
    the waiting launch shares its hardware queue with none of them, so no copy can end up behind it."""
    import torch
    dt, op, k, n, chunks = O.FP32, O.SUM, 3, 1 << 15, 24
    ins = make_inputs(dt, k, n * chunks, seed=31, op=op)
    staged = [to_dev(a) for a in ins]                       # where the producers read
    devs = [dev_empty(n * chunks, 4, fill=0) for _ in range(k)]  # where the reductions read
    out = dev_empty(n * chunks, 4, fill=0x55)
    others = [torch.cuda.Stream() for _ in range(12)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    with L.Gate() as gate:
        st = gate.own_stream()
        gate.reduce_batch([([d.data_ptr() + c * n * 4 for d in devs], out.data_ptr() + c * n * 4, n)
                           for c in range(chunks)], op, dt, k, stream=st)
        for c in range(chunks):
            s = others[(5 * c) % len(others)]
            with torch.cuda.stream(s):
                for j in range(k):
                    devs[j][c * n:(c + 1) * n].copy_(staged[j][c * n:(c + 1) * n])
            s.synchronize()
            gate.open(c + 1)
        assert L.lib().flagcxLocalGateOwnStream(gate._h, None) == L.Result.InvalidArgument
        import ctypes as C
        # the device adaptor's streamSynchronize, as the reference would synchronise a flagcxStream_t
        sync = L.adaptor_fn(L.device_adaptor()[1], "streamSynchronize", C.c_int, C.c_void_p)
        assert sync(C.addressof(st)) == 0
        assert gate.query() == (chunks, chunks, OK)
    assert time.perf_counter() - t0 < 1.0
    assert same(from_dev(out, np.float32), expect(ins, dt, op), nan_class=True, dtype=dt)


def test_numbers_start_at_zero_for_every_gate(L):
    """A gate's device word comes from a pool and goes on counting where its last gate stopped; the numbers a
    caller sees do not: each gate numbers its descriptors from 0 and reports its own count."""
    import torch
    dt, op, k, n = O.INT32, O.SUM, 2, 4099
    ins = make_inputs(dt, k, n, seed=41, op=op)
    devs = [to_dev(a) for a in ins]
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    for round_ in range(3):
        out = dev_empty(n, 4, fill=0x55)
        torch.cuda.synchronize()
        with L.Gate() as gate:
            assert gate.query() == (0, 0, OK)
            with torch.cuda.stream(side):
                first = gate.reduce_batch([([d.data_ptr() for d in devs], out.data_ptr(), n)] * 1, op, dt, k)
            assert first == 0
            gate.open(1 + round_)          # beyond what was launched: allowed
            side.synchronize()
            assert gate.query() == (1, 1 + round_, OK)
        assert same(from_dev(out, np.int32), expect(ins, dt, op), dtype=dt)
