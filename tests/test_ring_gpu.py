"""The staging ring: messages and reduce-scatter shards streamed through slots in
chunk steps on two streams must give the bytes of the direct calls."""
import ctypes as C

import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import dev_empty, from_dev, make_inputs, same, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    import torch
    assert torch.cuda.is_available()
    from flagcx_amd import local
    assert local.lib().flagcxLocalInit() == 0
    return local


def streams(L):
    import torch
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    return a, b, L.Stream(a.cuda_stream), L.Stream(b.cuda_stream)


@pytest.mark.parametrize("size,chunk,steps", [(1, 4096, 4), (4096 * 3, 4096, 4), (4096 * 37 + 100, 4096, 4),
                                              (1 << 20, 65536, 16), ((9 << 20) + 16, 0, 0),
                                              (4096 * 70 + 7, 4096, 8), (4096 * 40, 4096, 16)])   # steps in groups of half the ring, wraps
def test_ring_send_recv(L, size, chunk, steps):
    import torch
    ring_mem = torch.empty((steps or 16) * (chunk or L.CHUNKSIZE), dtype=torch.uint8, device="cuda")
    ring = L.Ring(ring_mem, 1, chunk, steps)
    h = np.random.default_rng(size).integers(0, 256, size, dtype=np.uint8)
    src = to_dev(h)
    dst = torch.full((size + 16,), 0x5A, dtype=torch.uint8, device="cuda")
    ta, tb, sa, sb = streams(L)
    torch.cuda.synchronize()
    ring.send_recv(dst.data_ptr(), src.data_ptr(), size, sa, sb)
    tb.synchronize()
    ta.synchronize()
    got = from_dev(dst, np.uint8)
    assert same(got[:size], h) and (got[size:] == 0x5A).all()
    ring.close()


@pytest.mark.parametrize("dt,op,nranks,rcount,chunk,steps", [
    (O.FP32, O.SUM, 4, 10000, 4096, 4),          # many wraps of a small ring, ragged last chunk
    (O.BF16, O.SUM, 8, 1 << 20, 1 << 18, 16),
    (O.FP16, O.AVG, 8, (1 << 21) + 24, 0, 0),     # default 16 x 4 MiB ring
    (O.INT32, O.MAX, 2, 5000, 4096, 2),
    (O.FP32, O.SUM, 8, 1024 * 37 + 25, 4096, 8),  # steps travel in groups of four here: many wraps, 37 whole steps + a ragged one
    (O.BF16, O.SUM, 8, 2048 * 70, 4096, 16),      # 70 whole steps, the last group of two
    (O.INT32, O.MIN, 5, 1024 * 9 + 1, 4096, 8),   # groups in a ring with every peer region in use, 5 ranks
])
def test_ring_reduce_scatter_equals_direct(L, dt, op, nranks, rcount, chunk, steps):
    import torch
    ts = O.type_size(dt)
    send_h = make_inputs(dt, nranks, nranks * rcount, seed=17 + dt, op=op)
    send = [to_dev(h) for h in send_h]
    ring_mem = torch.empty((steps or 16) * (nranks - 1) * (chunk or L.CHUNKSIZE), dtype=torch.uint8, device="cuda")
    ring = L.Ring(ring_mem, nranks - 1, chunk, steps)
    ta, tb, sa, sb = streams(L)
    for rank in (0, nranks - 1):
        direct = dev_empty(rcount, ts)
        staged = dev_empty(rcount, ts, fill=0)
        L.reduce_scatter(send, rank, direct, op, dtype=dt)
        torch.cuda.synchronize()
        ring.reduce_scatter(send, rank, staged, op, sa, sb, dtype=dt)
        tb.synchronize()
        ta.synchronize()
        assert torch.equal(direct, staged), rank
        rc, want = O.reduce_scatter_rank(send_h, rank, rcount, dt, op)
        nan_ok = dt in (O.FP16, O.BF16, O.FP32) and op in (O.SUM, O.AVG)
        assert same(from_dev(staged, send_h[0].dtype), want, nan_class=nan_ok, dtype=dt)
    ring.close()


@pytest.mark.parametrize("dt,op,nranks,rcount,chunk,steps", [
    (O.FP32, O.SUM, 4, 10000, 4096, 4),          # many wraps of a small ring, ragged last chunk
    (O.BF16, O.SUM, 8, 1 << 20, 1 << 18, 16),
    (O.FP16, O.AVG, 8, (1 << 21) + 24, 0, 0),     # default 16 x 4 MiB ring
    (O.INT32, O.MAX, 2, 5000, 4096, 2),
    (O.INT64, O.MIN, 3, 70001, 8192, 3),
    (O.FP32, O.SUM, 8, 1024 * 37 + 25, 4096, 8),  # grouped steps, many wraps, ragged end
    (O.BF16, O.SUM, 8, 2048 * 70, 4096, 16),
])
def test_ring_reduce_scatter_through_the_reduce_queue(L, dt, op, nranks, rcount, chunk, steps):
    """Proxy-style progress: copies on one stream, polled events, reduces through the
    resident consumer; same bytes as the direct call, for the first and the last rank,
    twice over on one ring and one running queue (slots and tickets are reused)."""
    import torch
    ts = O.type_size(dt)
    send_h = make_inputs(dt, nranks, nranks * rcount, seed=23 + dt, op=op)
    send = [to_dev(h) for h in send_h]
    ring_mem = torch.empty((steps or 16) * (nranks - 1) * (chunk or L.CHUNKSIZE), dtype=torch.uint8, device="cuda")
    ring = L.Ring(ring_mem, nranks - 1, chunk, steps)
    ta, tb, sa, sb = streams(L)
    direct = {rank: dev_empty(rcount, ts) for rank in (0, nranks - 1)}
    staged = {rank: dev_empty(rcount, ts, fill=0) for rank in (0, nranks - 1)}
    for rank in direct:
        L.reduce_scatter(send, rank, direct[rank], op, dtype=dt)
    torch.cuda.synchronize()
    L.lib().flagcxLocalSetMaxSpinCount(1 << 19)
    q = L.ReduceFifo(8, nranks, dt, op)
    try:
        # the copy stream must not sit behind the consumer, however many streams this process has made before
        q.set_own_queue(True)
        with q:
            for rep in range(2):
                for rank in staged:
                    ring.reduce_scatter_fifo(q, send, rank, staged[rank], sa)
                    assert q.query()[2] in (1, 4)
    finally:
        q.close()
        L.lib().flagcxLocalSetMaxSpinCount(-1)
    torch.cuda.synchronize()
    for rank in staged:
        assert torch.equal(direct[rank], staged[rank]), rank
        rc, want = O.reduce_scatter_rank(send_h, rank, rcount, dt, op)
        nan_ok = dt in (O.FP16, O.BF16, O.FP32) and op in (O.SUM, O.AVG)
        assert same(from_dev(staged[rank], send_h[0].dtype), want, nan_class=nan_ok, dtype=dt)
    ring.close()


def test_ring_rejects_bad_arguments(L):
    import torch
    mem = torch.empty(1 << 20, dtype=torch.uint8, device="cuda")
    h = C.c_void_p()
    lib = L.lib()
    inv = int(L.Result.InvalidArgument)
    assert lib.flagcxLocalRingCreate(C.byref(h), mem.data_ptr(), 1 << 20, 1, 0, 0) == inv      # 64 MiB needed
    assert lib.flagcxLocalRingCreate(C.byref(h), mem.data_ptr(), 1 << 20, 0, 4096, 4) == inv
    assert lib.flagcxLocalRingCreate(C.byref(h), mem.data_ptr(), 1 << 20, 1, 4100, 4) == inv   # chunk % 16
    assert lib.flagcxLocalRingCreate(C.byref(h), None, 1 << 20, 1, 4096, 4) == inv
    assert lib.flagcxLocalRingCreate(C.byref(h), mem.data_ptr(), 1 << 20, 1, 4096, 4) == 0
    st = L.current_stream()
    assert lib.flagcxLocalRingSendRecv(h, mem.data_ptr(), mem.data_ptr() + 4096, 16, None, C.byref(st)) == inv
    ptrs = (C.c_void_p * 3)(mem.data_ptr(), mem.data_ptr(), mem.data_ptr())
    assert lib.flagcxLocalRingReduceScatter(h, ptrs, 3, 0, mem.data_ptr(), 16, 7, 0, C.byref(st), C.byref(st)) == inv
    assert lib.flagcxLocalRingDestroy(h) == 0


def test_ring_fifo_returns_when_the_consumer_has_left(L):
    """A consumer that gives up on its spin bound while the host still waits for ring
    slots: the call returns an error instead of waiting for `consumed` to move, every
    kernel having ended normally, and the same queue works again after a restart.
    (With a spin bound of one poll the consumer leaves at the first entry it cannot
    finish between two polls; should it get through all the same, the bytes are right.)"""
    import torch
    dt, op, nranks, rcount, chunk, steps = O.FP32, O.SUM, 4, 4096 * 64, 4096, 2
    ts = O.type_size(dt)
    send_h = make_inputs(dt, nranks, nranks * rcount, seed=99, op=op)
    send = [to_dev(h) for h in send_h]
    ring_mem = torch.empty(steps * (nranks - 1) * chunk, dtype=torch.uint8, device="cuda")
    ring = L.Ring(ring_mem, nranks - 1, chunk, steps)
    ta, tb, sa, sb = streams(L)
    out = dev_empty(rcount, ts, fill=0)
    rc, want = O.reduce_scatter_rank(send_h, 1, rcount, dt, op)
    torch.cuda.synchronize()
    q = L.ReduceFifo(8, nranks, dt, op)
    try:
        q.set_own_queue(True)  # the copy stream never waits behind the consumer
        # the spin bound is reached long before the idle limit at which a consumer parks
        L.lib().flagcxLocalSetMaxSpinCount(1)
        q.start()
        try:
            ring.reduce_scatter_fifo(q, send, 1, out, sa)
            left = False
        except L.FlagcxError:
            left = True
        torch.cuda.synchronize()              # returns: no kernel is left spinning
        if left:
            assert q.query()[2] == 3          # timed out
            try:
                q.stop()
            except L.FlagcxError:
                pass                          # reports the entries that were not reached
        else:
            q.stop()
            assert same(from_dev(out, send_h[0].dtype), want, nan_class=True, dtype=dt)
        L.lib().flagcxLocalSetMaxSpinCount(1 << 19)
        out.zero_()
        torch.cuda.synchronize()
        with q:
            ring.reduce_scatter_fifo(q, send, 1, out, sa)
        assert same(from_dev(out, send_h[0].dtype), want, nan_class=True, dtype=dt)
    finally:
        L.lib().flagcxLocalSetMaxSpinCount(-1)
        q.close()
        ring.close()


@pytest.mark.parametrize("size,chunk,steps", [(4096 * 9 + 5, 4096, 4), (1 << 20, 65536, 16)])
def test_ring_send_recv_through_a_host_bounce_buffer(L, size, chunk, steps):
    """The socket transport's variant of the staging steps (flagcx/core/net.cc:153-161,
    298-306): the ring is pinned host memory, so the producer's copies are device-to-host
    and the consumer's host-to-device, done by the same copy kernels over PCIe."""
    import torch
    ring_mem = torch.empty(steps * chunk, dtype=torch.uint8, pin_memory=True)
    ring = L.Ring(ring_mem, 1, chunk, steps)
    h = np.random.default_rng(size).integers(0, 256, size, dtype=np.uint8)
    src = to_dev(h)
    dst = torch.full((size + 16,), 0x5A, dtype=torch.uint8, device="cuda")
    ta, tb, sa, sb = streams(L)
    torch.cuda.synchronize()
    ring.send_recv(dst.data_ptr(), src.data_ptr(), size, sa, sb)
    tb.synchronize()
    ta.synchronize()
    got = from_dev(dst, np.uint8)
    assert same(got[:size], h) and (got[size:] == 0x5A).all()
    ring.close()
