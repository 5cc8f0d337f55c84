"""flagcxLocalStagedReduceScatterNoAlloc - the entry point for callers that cannot
allocate - against the existing flagcxLocalRingReduceScatter (caller's ring buffer,
ring object, two streams), bit for bit, through the C ABI; and against the oracle.
Two calls in a row share the library's one staging area, the second one smaller."""
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


def ring_result(L, send, rank, rcount, dt, op, ts):
    """What the existing entry point gives: 16 slots of 64 KiB on two streams."""
    import torch
    nranks = len(send)
    chunk, steps = 65536, 16
    ring_mem = torch.empty(steps * max(nranks - 1, 1) * chunk, dtype=torch.uint8, device="cuda")
    ring = L.Ring(ring_mem, max(nranks - 1, 1), chunk, steps)
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    out = dev_empty(rcount, ts, fill=0)
    torch.cuda.synchronize()
    ring.reduce_scatter(send, rank, out, op, L.Stream(a.cuda_stream), L.Stream(b.cuda_stream), dtype=dt)
    b.synchronize()
    a.synchronize()
    ring.close()
    return out


def staged(L, send, rank, out, op, dt):
    L.staged_reduce_scatter_noalloc(send, rank, out, op, dtype=dt)


CASES = [
    # dtype, op, nranks, first recvcount, second (smaller) recvcount
    (O.BF16, O.SUM, 8, 500000, 70001),      # 7 peers x ~1 MB: most of the area, then a ragged small one
    (O.FP32, O.SUM, 4, 300000 + 3, 1000),
    (O.FP16, O.AVG, 8, 1 << 18, 33),
    (O.INT32, O.MAX, 2, 2000000, 5),        # one peer, ~8 MB: just inside the limit
    (O.INT64, O.MIN, 3, 70001, 7),
    (O.UINT8, O.SUM, 5, 12345, 1),
]


@pytest.mark.parametrize("dt,op,nranks,first,second", CASES)
def test_no_alloc_entry_point_matches_the_ring_entry_point(L, dt, op, nranks, first, second):
    import torch
    ts = O.type_size(dt)
    nan_ok = dt in (O.FP16, O.BF16, O.FP32) and op in (O.SUM, O.AVG)
    for call, rcount in enumerate((first, second)):      # two calls in a row, the second smaller
        send_h = make_inputs(dt, nranks, nranks * rcount, seed=31 + dt + call, op=op)
        send = [to_dev(h) for h in send_h]
        for rank in (0, nranks - 1):
            want_dev = ring_result(L, send, rank, rcount, dt, op, ts)
            got = dev_empty(rcount + 8, ts, fill=0x5A)
            staged(L, send, rank, got[:rcount], op, dt)
            torch.cuda.synchronize()
            assert torch.equal(got[:rcount], want_dev), (call, rank)
            assert bool((got[rcount:] == 0x5A).all()), "wrote past the shard"
            rc, want = O.reduce_scatter_rank(send_h, rank, rcount, dt, op)
            assert rc == 0
            assert same(from_dev(got[:rcount], send_h[0].dtype), want, nan_class=nan_ok, dtype=dt), (call, rank)


def test_no_alloc_entry_point_unaligned_output_and_in_place(L):
    """recvbuff at an odd element offset (regions follow its offset inside a 16-byte
    line), and recvbuff == the local slice (in place)."""
    import torch
    dt, op, nranks, rcount = O.FP32, O.SUM, 4, 4099
    send_h = make_inputs(dt, nranks, nranks * rcount, seed=77, op=op)
    for rank in range(nranks):
        send = [to_dev(h) for h in send_h]
        rc, want = O.reduce_scatter_rank(send_h, rank, rcount, dt, op)
        out = dev_empty(rcount + 3, 4, fill=0)
        staged(L, send, rank, out[3:], op, dt)
        torch.cuda.synchronize()
        assert same(from_dev(out[3:], np.float32), want, nan_class=True, dtype=dt), rank
        local = send[rank][rank * rcount:(rank + 1) * rcount]
        staged(L, send, rank, local, op, dt)
        torch.cuda.synchronize()
        assert same(from_dev(local, np.float32), want, nan_class=True, dtype=dt), rank


def test_no_alloc_entry_point_one_rank_is_a_copy(L):
    import torch
    h = make_inputs(O.FP16, 1, 5000, seed=5)[0]
    src = to_dev(h)
    out = dev_empty(5000, 2, fill=0)
    staged(L, [src], 0, out, O.SUM, O.FP16)
    torch.cuda.synchronize()
    assert torch.equal(out, src)


def test_no_alloc_entry_point_rejects_what_does_not_fit(L):
    import torch
    lib = L.lib()
    inv = int(L.Result.InvalidArgument)
    limit = L.STATIC_STAGING_BYTES
    mem = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    st = L.current_stream()

    def call(ptrs, n, rank, dst, count, dtype=7, op=0):
        arr = (C.c_void_p * len(ptrs))(*ptrs)
        return lib.flagcxLocalStagedReduceScatterNoAlloc(arr, n, rank, dst, count, dtype, op, C.byref(st))

    p = mem.data_ptr()
    # 1 peer x (limit + 4) bytes, 7 peers x limit / 4 bytes: never dereferenced, validation fails first
    assert call([p, p], 2, 0, p + 2048, limit // 4 + 1) == inv
    assert b"static staging area" in lib.flagcxLocalGetLastError()
    assert call([p] * 8, 8, 0, p + 2048, limit // 16) == inv
    assert b"static staging area" in lib.flagcxLocalGetLastError()
    assert call([p, p], 2, 0, p + 2048, 16, dtype=10) == inv
    assert call([p, p], 2, 0, p + 2048, 16, op=5) == inv
    assert call([p, p], 2, 2, p + 2048, 16) == inv
    assert call([p, 0], 2, 0, p + 2048, 16) == inv
    assert call([p, p], 2, 0, 0, 16) == inv
    assert call([p, p + 1024], 2, 0, p + 8, 16) == inv           # output overlaps a slice that is read
    assert call([p, p + 1024], 2, 0, p + 2048, 0) == 0           # nothing to do
    torch.cuda.synchronize()


def test_no_alloc_entry_point_under_stream_capture_and_without_taking_memory(L):
    """What the entry point is for.  Captured between hipStreamBeginCapture and
    hipStreamEndCapture (a call that allocated, freed or synchronised there would end the
    capture with an error: the capture mode is the strict one), then replayed four times over
    new inputs with eager work in between, every replay against the oracle, the second shape
    smaller than the first; and the device's free memory is the same before and after the calls."""
    import torch
    dt, op, nranks = O.BF16, O.SUM, 8
    ts = O.type_size(dt)
    side = torch.cuda.Stream()
    for rcount in (200000 + 5, 4099):
        send_h = make_inputs(dt, nranks, nranks * rcount, seed=91 + rcount % 7, op=op)
        send = [to_dev(h) for h in send_h]
        out = dev_empty(rcount + 8, ts, fill=0x5A)
        rank = 5
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            staged(L, send, rank, out[:rcount], op, dt)        # eager once on the capture stream
        side.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side, capture_error_mode="global"):
            staged(L, send, rank, out[:rcount], op, dt)
        for rep in range(4):
            perm = np.roll(np.arange(nranks), rep + 1)
            for j in range(nranks):
                send[j].copy_(to_dev(send_h[perm[j]]))
            out.fill_(0x5A5A)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            rc, want = O.reduce_scatter_rank([send_h[perm[j]] for j in range(nranks)], rank, rcount, dt, op)
            assert rc == 0
            assert same(from_dev(out[:rcount], np.uint16), want, nan_class=True, dtype=dt), (rcount, rep)
            assert bool((out[rcount:] == 0x5A5A).all()), "wrote past the shard"
        # eager calls take no device memory either
        for _ in range(3):
            staged(L, send, rank, out[:rcount], op, dt)
        torch.cuda.synchronize()
        del g
        assert torch.cuda.mem_get_info()[0] >= free_before, "the calls took device memory"
