"""Re-entrancy of the C ABI: the reference enters its device layer from user threads,
from the per-communicator proxy thread on its own stream (flagcx/core/proxy.cc:365-378,
flagcx/core/p2p.cc:86-91) and from the kernel-proxy thread (proxy.cc:1074-1099), so
every entry point must work from several threads at once, on streams made elsewhere."""
import threading

import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import dev_empty, from_dev, make_inputs, same, to_dev


@pytest.mark.gpu
def test_concurrent_callers_on_their_own_streams():
    import torch
    from flagcx_amd import local as L
    assert L.lib().flagcxLocalInit() == 0
    nthreads, rounds = 6, 40
    cases = [(O.BF16, O.SUM, 8), (O.FP32, O.SUM, 2), (O.INT32, O.MAX, 4), (O.FP16, O.AVG, 3), (O.INT64, O.MIN, 5),
             (O.UINT8, O.PROD, 2)]
    n = 200_003
    work = []
    for t in range(nthreads):
        dt, op, k = cases[t]
        ins = make_inputs(dt, k, n, seed=40 + t, op=op)
        work.append((dt, op, ins, [to_dev(a) for a in ins], dev_empty(n, ins[0].dtype.itemsize, fill=0),
                     dev_empty(n, ins[0].dtype.itemsize, fill=0)))
    # streams are created here, on the main thread, and used from the workers
    streams = [torch.cuda.Stream() for _ in range(nthreads)]
    torch.cuda.synchronize()
    errors = []
    barrier = threading.Barrier(nthreads)

    def run(t):
        try:
            dt, op, ins, devs, out, packed = work[t]
            st = L.Stream(streams[t].cuda_stream)
            barrier.wait()
            for r in range(rounds):
                L.reduce(devs, out, op, dtype=dt, stream=st)
                L.memcpy(packed.data_ptr(), out.data_ptr(), n * ins[0].dtype.itemsize, stream=st)
                if r % 8 == 0:
                    # a deliberate error on this thread must not show up on the others
                    rc = L.lib().flagcxLocalReduce(None, 2, None, 16, int(dt), int(op), None)
                    assert rc == int(L.Result.InvalidArgument)
                    assert b"flagcxLocalReduce" in L.lib().flagcxLocalGetLastError()
            streams[t].synchronize()
        except Exception as e:  # collected and re-raised on the main thread
            errors.append((t, repr(e)))

    threads = [threading.Thread(target=run, args=(t,)) for t in range(nthreads)]
    for th in threads:
        th.start()
    for th in threads:
        th.join(120)
    assert not errors, errors
    torch.cuda.synchronize()
    for t in range(nthreads):
        dt, op, ins, devs, out, packed = work[t]
        rc, want = O.reduce(ins, dt, op)
        assert rc == 0
        nan = dt in (O.BF16, O.FP16, O.FP32)
        assert same(from_dev(out, ins[0].dtype), want, nan_class=nan, dtype=dt), t
        assert same(from_dev(packed, ins[0].dtype), want, nan_class=nan, dtype=dt), t


def test_last_error_is_per_thread():
    from flagcx_amd import local as L
    lib = L.lib()
    seen = {}

    def bad():
        lib.flagcxLocalReduce(None, 99, None, 16, 7, 0, None)
        seen["bad"] = lib.flagcxLocalGetLastError()

    def clean():
        seen["clean"] = lib.flagcxLocalGetLastError()

    a = threading.Thread(target=bad)
    a.start()
    a.join()
    b = threading.Thread(target=clean)
    b.start()
    b.join()
    assert b"sendbuffs is NULL" in seen["bad"]
    assert seen["clean"] == b""


def test_tuning_overrides_belong_to_the_calling_thread():
    """flagcxLocalTune / flagcxLocalTuneLoads shape the launches of the thread that set
    them: another thread still sees (and launches with) the library's own choice."""
    import ctypes as C
    from flagcx_amd import local as L
    lib = L.lib()
    seen = {}
    ready, done = threading.Event(), threading.Event()

    def tuner():
        assert lib.flagcxLocalTune(8, 25) == 0 and lib.flagcxLocalTuneLoads(8, 1) == 0
        w, l = C.c_int(-2), C.c_int(-2)
        assert lib.flagcxLocalGetTune(8, C.byref(w)) == 0 and lib.flagcxLocalGetTuneLoads(8, C.byref(l)) == 0
        seen["tuner"] = (w.value, l.value)
        ready.set()
        done.wait(30)
        # still set here after the other thread has looked and set its own
        assert lib.flagcxLocalGetTune(8, C.byref(w)) == 0 and lib.flagcxLocalGetTuneLoads(8, C.byref(l)) == 0
        seen["tuner_after"] = (w.value, l.value)

    def other():
        ready.wait(30)
        w, l = C.c_int(-2), C.c_int(-2)
        assert lib.flagcxLocalGetTune(8, C.byref(w)) == 0 and lib.flagcxLocalGetTuneLoads(8, C.byref(l)) == 0
        seen["other"] = (w.value, l.value)
        assert lib.flagcxLocalTune(8, 10) == 0
        done.set()

    a, b = threading.Thread(target=tuner), threading.Thread(target=other)
    a.start()
    b.start()
    a.join(60)
    b.join(60)
    assert seen == {"tuner": (25, 1), "other": (-1, -1), "tuner_after": (25, 1)}
    w = C.c_int(-2)
    assert lib.flagcxLocalGetTune(8, C.byref(w)) == 0 and w.value == -1     # and the main thread was never touched


@pytest.mark.gpu
def test_queue_gate_and_plain_launches_side_by_side():
    """The three ways into the reduce at once, each from its own thread: entries through the resident queue
    (on a hardware queue of its own), gated batches on the gate's own stream opened chunk by chunk, and plain
    launches on an ordinary stream.  Whatever the runtime's mapping of streams to hardware queues, neither of
    the two kernels that wait on the GPU can hold the third thread's stream up for good, and every result is
    the oracle's."""
    import time
    import torch
    from flagcx_amd import local as L
    assert L.lib().flagcxLocalInit() == 0
    L.lib().flagcxLocalSetMaxSpinCount(1 << 21)
    n, rounds = 1 << 16, 12
    mk = lambda dt, op, k, seed: make_inputs(dt, k, n * rounds, seed=seed, op=op)
    qi, gi, pi = mk(O.FP16, O.AVG, 8, 1), mk(O.FP32, O.SUM, 3, 2), mk(O.INT32, O.MAX, 4, 3)
    qd, gd, pd = ([to_dev(a) for a in x] for x in (qi, gi, pi))
    qo, go, po = dev_empty(n * rounds, 2, fill=0), dev_empty(n * rounds, 4, fill=0), dev_empty(n * rounds, 4, fill=0)
    plain = torch.cuda.Stream()
    torch.cuda.synchronize()
    errors = []
    barrier = threading.Barrier(3)

    def through_queue():
        try:
            q = L.ReduceFifo(16, 8, O.FP16, O.AVG)
            try:
                q.set_own_queue(True)
                with q:
                    barrier.wait()
                    t = 0
                    for r in range(rounds):
                        t = q.enqueue_reduce([d.data_ptr() + r * n * 2 for d in qd], qo.data_ptr() + r * n * 2, n)
                        time.sleep(0.0005)
                    q.wait(t)
            finally:
                q.close()
        except Exception as e:
            errors.append(("queue", repr(e)))

    def through_gate():
        try:
            with L.Gate() as gate:
                st = gate.own_stream()
                barrier.wait()
                first = gate.reduce_batch([([d.data_ptr() + r * n * 4 for d in gd], go.data_ptr() + r * n * 4, n)
                                           for r in range(rounds)], O.SUM, O.FP32, 3, stream=st)
                for r in range(rounds):
                    time.sleep(0.0005)
                    gate.open(first + r + 1)
                import ctypes as C
                sync = L.adaptor_fn(L.device_adaptor()[1], "streamSynchronize", C.c_int, C.c_void_p)
                assert sync(C.addressof(st)) == 0
                assert gate.query()[2] == 0
        except Exception as e:
            errors.append(("gate", repr(e)))

    def plain_launches():
        try:
            st = L.Stream(plain.cuda_stream)
            barrier.wait()
            for r in range(rounds):
                L.reduce([d[r * n:(r + 1) * n] for d in pd], po[r * n:(r + 1) * n], O.MAX, dtype=O.INT32, stream=st)
                time.sleep(0.0005)
            plain.synchronize()
        except Exception as e:
            errors.append(("plain", repr(e)))

    threads = [threading.Thread(target=f) for f in (through_queue, through_gate, plain_launches)]
    try:
        for th in threads:
            th.start()
        for th in threads:
            th.join(60)
    finally:
        L.lib().flagcxLocalSetMaxSpinCount(-1)
    assert not errors, errors
    assert not any(th.is_alive() for th in threads)
    torch.cuda.synchronize()
    for ins, out, dt, op in ((qi, qo, O.FP16, O.AVG), (gi, go, O.FP32, O.SUM), (pi, po, O.INT32, O.MAX)):
        rc, want = O.reduce(ins, dt, op)
        assert rc == 0
        assert same(from_dev(out, ins[0].dtype), want, nan_class=dt != O.INT32, dtype=dt), (dt, op)


@pytest.mark.gpu
def test_two_gates_waiting_at_once_and_a_plain_launch_behind_them():
    """Two gated batches wait on the GPU at the same time, each on its gate's own stream and each large
    enough to fill its share of every CU's wavefront slots (8 chunks of 1024 tiles), and a plain launch is
    enqueued on a third stream while both wait.  The host opens the gates chunk by chunk, the second gate
    first; nothing the GPU holds can keep the host from doing so, so all three finish, with the oracle's
    bytes.  The waits are bounded by the spin limit, as in every test of a waiting kernel."""
    import ctypes as C
    import torch
    from flagcx_amd import local as L
    assert L.lib().flagcxLocalInit() == 0
    L.lib().flagcxLocalSetMaxSpinCount(1 << 22)
    try:
        n, chunks = 1 << 19, 8
        ai, bi, pi = (make_inputs(dt, k, n * chunks, seed=s, op=op) for dt, k, s, op in
                      ((O.FP16, 4, 11, O.AVG), (O.BF16, 8, 12, O.SUM), (O.INT32, 3, 13, O.MIN)))
        ad, bd, pd = ([to_dev(a) for a in x] for x in (ai, bi, pi))
        ao, bo, po = dev_empty(n * chunks, 2, fill=0), dev_empty(n * chunks, 2, fill=0), dev_empty(n * chunks, 4, fill=0)
        plain = torch.cuda.Stream()
        torch.cuda.synchronize()
        sync = L.adaptor_fn(L.device_adaptor()[1], "streamSynchronize", C.c_int, C.c_void_p)
        with L.Gate() as ga, L.Gate() as gb:
            sa, sb = ga.own_stream(), gb.own_stream()
            fa = ga.reduce_batch([([d.data_ptr() + c * n * 2 for d in ad], ao.data_ptr() + c * n * 2, n)
                                  for c in range(chunks)], O.AVG, O.FP16, 4, stream=sa)
            fb = gb.reduce_batch([([d.data_ptr() + c * n * 2 for d in bd], bo.data_ptr() + c * n * 2, n)
                                  for c in range(chunks)], O.SUM, O.BF16, 8, stream=sb)
            L.reduce(pd, po, O.MIN, dtype=O.INT32, stream=L.Stream(plain.cuda_stream))
            for c in range(chunks):
                gb.open(fb + c + 1)
                if c % 2:
                    ga.open(fa + c + 1)            # the first gate two chunks at a time
            assert sync(C.addressof(sb)) == 0 and sync(C.addressof(sa)) == 0
            plain.synchronize()
            assert ga.query()[2] == 0 and gb.query()[2] == 0
        torch.cuda.synchronize()
        for ins, out, dt, op in ((ai, ao, O.FP16, O.AVG), (bi, bo, O.BF16, O.SUM), (pi, po, O.INT32, O.MIN)):
            rc, want = O.reduce(ins, dt, op)
            assert rc == 0
            assert same(from_dev(out, ins[0].dtype), want, nan_class=dt != O.INT32, dtype=dt), (dt, op)
    finally:
        L.lib().flagcxLocalSetMaxSpinCount(-1)
