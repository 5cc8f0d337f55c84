"""GPU parity of the chunk copy / pack / unpack / fill kernels: byte-exact against
the oracle's memcpy loops, round trips, and untouched guard bytes."""
import ctypes as C

import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import from_dev, same, to_dev

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    import torch
    assert torch.cuda.is_available()
    from flagcx_amd import local
    assert local.lib().flagcxLocalInit() == 0
    return local


def rand_bytes(n, seed):
    return np.random.default_rng(seed).integers(0, 256, n, dtype=np.uint8)


@pytest.mark.parametrize("size", [1, 15, 16, 17, 1000, 4096, 65536 + 5, (4 << 20), (4 << 20) + 123])
def test_memcpy_sizes_and_offsets(L, size):
    import torch
    src_h = rand_bytes(size + 64, size)
    src = to_dev(src_h)
    # the last four: 16-byte aligned on both sides but inside a 128-byte line (short first tile)
    for so, do in ((0, 0), (1, 1), (3, 3), (0, 5), (7, 2), (4, 8), (2, 4), (16, 16), (0, 48), (32, 0), (19, 35)):
        dst = torch.full((size + 64,), 0xAB, dtype=torch.uint8, device="cuda")
        L.memcpy(dst.data_ptr() + do, src.data_ptr() + so, size)
        torch.cuda.synchronize()
        got = from_dev(dst, np.uint8)
        assert same(got[do:do + size], src_h[so:so + size]), (so, do)
        assert (got[:do] == 0xAB).all() and (got[do + size:] == 0xAB).all(), (so, do)


def test_self_copy_reference_pattern(L):
    # test/perf/test_core_sendrecv.cpp:80-94: 0xAA x 100 then 0xBB x 200, self send/recv
    import torch
    h = np.concatenate([np.full(100, 0xAA, np.uint8), np.full(200, 0xBB, np.uint8)])
    src = to_dev(h)
    dst = torch.zeros(300, dtype=torch.uint8, device="cuda")
    args = L.CopyArgs(dst.data_ptr(), src.data_ptr(), 300, -1, 0)
    st = L.current_stream()
    L.lib().flagcxLocalCopyFunc(C.byref(st), C.byref(args))
    torch.cuda.synchronize()
    assert args.result == 0 and same(from_dev(dst, np.uint8), h)


@pytest.mark.parametrize("size", [1, 31, 4096, 100003])
def test_memset(L, size):
    import torch
    for off, val in ((0, 0), (1, 0x5A), (9, 0xFF), (16, 7), (48, 3), (35, 9)):
        buf = torch.full((size + 64,), 0xCD, dtype=torch.uint8, device="cuda")
        L.memset(buf.data_ptr() + off, val, size)
        torch.cuda.synchronize()
        got = from_dev(buf, np.uint8)
        assert (got[off:off + size] == val).all()
        assert (got[:off] == 0xCD).all() and (got[off + size:] == 0xCD).all()


@pytest.mark.parametrize("tsz,dt", [(4, O.FP32), (2, O.BF16), (1, O.INT8), (8, O.FP64)])
def test_refresh_matches_oracle(L, tsz, dt):
    import torch
    carrier = {1: np.uint8, 2: np.uint16, 4: np.float32, 8: np.float64}[tsz]
    for start, offset, count, total in ((0, 0, 10, 100), (3, 20, 30, 80), (0, 90, 10, 100), (5, 0, 0, 50),
                                        (1, 1000, 3000, 100001), (0, 7, 1, 9)):
        n = start + total + 13
        h = rand_bytes(n * tsz, total).view(carrier).copy()
        for op in (O.SUM, O.MAX, O.MIN, O.PROD):
            want = h.copy()
            O.refresh(want, start, offset, count, total, op)
            d = to_dev(h)
            L.refresh(d, start, offset, count, total, op, dtype=dt)
            torch.cuda.synchronize()
            assert same(from_dev(d, carrier), want), (start, offset, count, total, op)


@pytest.mark.parametrize("chunk,stride", [(64, 512), (4096, 32768), (100, 800), (48, 48), (17, 33),
                                          (1 << 20, 8 << 20), (6, 64), (4096 + 16, 8192 + 48), (2048, 4096 + 16)])
def test_pack_unpack_round_trip(L, chunk, stride):
    import torch
    nch = 8
    span = (nch - 1) * stride + chunk
    h = rand_bytes(span + 32, chunk + stride)
    for base in (0, 4, 1, 16):  # 16: vector path with every chunk inside a 128-byte line
        src = to_dev(h)
        staged = torch.full((nch * chunk + 32,), 0x77, dtype=torch.uint8, device="cuda")
        L.pack(staged.data_ptr() + base, src.data_ptr() + base, nch, chunk, stride)
        torch.cuda.synchronize()
        want = O.pack(np.ascontiguousarray(h[base:]), nch, chunk, stride)
        got = from_dev(staged, np.uint8)
        assert same(got[base:base + nch * chunk], want), (chunk, stride, base)
        assert (got[:base] == 0x77).all() and (got[base + nch * chunk:] == 0x77).all()
        # scatter back into a fresh sparse buffer: chunks restored, gaps untouched
        back = torch.full((span + 32,), 0xEE, dtype=torch.uint8, device="cuda")
        L.unpack(back.data_ptr() + base, staged.data_ptr() + base, nch, chunk, stride)
        torch.cuda.synchronize()
        wantb = np.full(span + 32, 0xEE, np.uint8)
        O.unpack(wantb[base:], want, nch, chunk, stride)
        assert same(from_dev(back, np.uint8), wantb), (chunk, stride, base)


@pytest.mark.parametrize("nch,cb,gap,so,do", [
    (37, 4099, 3, 5, 9),        # nothing is a multiple of 16: every chunk has head and tail bytes of its own, sources shifted
    (64, 1024, 1, 0, 1),        # the shortest chunks that take the vector body
    (64, 70001, 0, 3, 3),       # contiguous chunks, both sides at the same odd offset
    (200, 2049, 77, 1, 2),
    (3, 1 << 20, 16, 8, 0),     # 16-byte strides, the two sides 8 bytes apart
    (9, 1023, 5, 7, 11),        # one tile per chunk
    (300, 321, 2, 3, 1),        # many chunks just long enough for the vector body, one workgroup each
    (9, 300, 5, 7, 11),         # shorter than that: the element path
])
def test_pack_unpack_ragged_chunks(L, nch, cb, gap, so, do):
    """Strided chunks whose size, stride and bases are no multiples of 16: packed, and unpacked
    again at another stride, byte-exact against numpy slices, guard bytes untouched."""
    import torch
    stride = cb + gap
    sparse_h = rand_bytes(so + nch * stride + 64, nch * 131 + cb)
    want = np.concatenate([sparse_h[so + i * stride:so + i * stride + cb] for i in range(nch)])
    sparse = to_dev(sparse_h)
    packed = torch.full((do + nch * cb + 64,), 0xAB, dtype=torch.uint8, device="cuda")
    L.pack(packed.data_ptr() + do, sparse.data_ptr() + so, nch, cb, stride)
    torch.cuda.synchronize()
    got = from_dev(packed, np.uint8)
    assert same(got[do:do + nch * cb], want)
    assert (got[:do] == 0xAB).all() and (got[do + nch * cb:] == 0xAB).all()
    stride2 = cb + 2 * gap + 1
    out = torch.full((so + nch * stride2 + 64,), 0xCD, dtype=torch.uint8, device="cuda")
    L.unpack(out.data_ptr() + so, packed.data_ptr() + do, nch, cb, stride2)
    torch.cuda.synchronize()
    got = from_dev(out, np.uint8)
    expect = np.full(got.shape, 0xCD, np.uint8)
    for i in range(nch):
        expect[so + i * stride2:so + i * stride2 + cb] = want[i * cb:(i + 1) * cb]
    assert same(got, expect)


def test_pack_list_and_unpack_list_of_64_ragged_entries(L):
    """The most entries a list takes, each at a position of its own inside a cache line."""
    import torch
    n, cb = 64, 5003
    rng = np.random.default_rng(64)
    offs = [int(x) for x in rng.integers(0, 128, n)]
    hosts = [rand_bytes(cb + 256, 900 + i) for i in range(n)]
    want = np.concatenate([hosts[i][offs[i]:offs[i] + cb] for i in range(n)])
    srcs = [to_dev(h) for h in hosts]
    packed = torch.full((n * cb + 64,), 0xAB, dtype=torch.uint8, device="cuda")
    L.pack_list(packed.data_ptr() + 3, [s.data_ptr() + o for s, o in zip(srcs, offs)], cb)
    torch.cuda.synchronize()
    got = from_dev(packed, np.uint8)
    assert same(got[3:3 + n * cb], want) and (got[:3] == 0xAB).all() and (got[3 + n * cb:] == 0xAB).all()
    dsts = [torch.full((cb + 256,), 0xCD, dtype=torch.uint8, device="cuda") for _ in range(n)]
    offs2 = [int(x) for x in rng.integers(0, 128, n)]
    L.unpack_list([d.data_ptr() + o for d, o in zip(dsts, offs2)], packed.data_ptr() + 3, cb)
    torch.cuda.synchronize()
    for i, d in enumerate(dsts):
        g = from_dev(d, np.uint8)
        assert same(g[offs2[i]:offs2[i] + cb], want[i * cb:(i + 1) * cb]), i
        assert (g[:offs2[i]] == 0xCD).all() and (g[offs2[i] + cb:] == 0xCD).all(), i


@pytest.mark.parametrize("nbytes", [16, 1000, 4096, 65536 + 16, 333])
def test_pack_list_and_unpack_list(L, nbytes):
    import torch
    n = 8
    hs = [rand_bytes(nbytes + 16, 100 + j) for j in range(n)]
    for off in (0, 3):
        devs = [to_dev(h) for h in hs]
        flat = torch.full((n * nbytes + 16,), 0x11, dtype=torch.uint8, device="cuda")
        L.pack_list(flat.data_ptr() + off, [d.data_ptr() + off for d in devs], nbytes)
        torch.cuda.synchronize()
        got = from_dev(flat, np.uint8)
        want = np.concatenate([h[off:off + nbytes] for h in hs])
        assert same(got[off:off + n * nbytes], want), (nbytes, off)
        assert (got[:off] == 0x11).all() and (got[off + n * nbytes:] == 0x11).all()
        outs = [torch.full((nbytes + 16,), 0x22, dtype=torch.uint8, device="cuda") for _ in range(n)]
        L.unpack_list([o.data_ptr() + off for o in outs], flat.data_ptr() + off, nbytes)
        torch.cuda.synchronize()
        for j in range(n):
            g = from_dev(outs[j], np.uint8)
            assert same(g[off:off + nbytes], hs[j][off:off + nbytes]), (nbytes, off, j)
            assert (g[:off] == 0x22).all() and (g[off + nbytes:] == 0x22).all()


@pytest.mark.parametrize("size", [1, 15, 16, 17, 1000, 4096, 65536 + 5, (3 << 20) + 77])
def test_copy_fanout_sizes_offsets_and_destination_counts(L, size):
    """One source to 1..11 destinations (more than eight share the source in two reads), at
    offsets that agree with the source modulo 16 (inside and on 128-byte lines) and at
    offsets that do not (those go as plain copies); bytes and guard bytes of every
    destination against numpy."""
    import torch
    rng = np.random.default_rng(size)
    src_h = rand_bytes(size + 256, size)
    src = to_dev(src_h)
    for so, ndst in ((0, 1), (0, 4), (3, 3), (16, 8), (5, 11), (64, 2), (130, 5)):
        dos = [so + 16 * int(rng.integers(0, 8)) if j % 3 != 2 else int(rng.integers(0, 200)) for j in range(ndst)]
        dsts = [torch.full((size + 512,), 0xAB, dtype=torch.uint8, device="cuda") for _ in range(ndst)]
        L.copy_fanout([(src.data_ptr() + so, [d.data_ptr() + o for d, o in zip(dsts, dos)], size)])
        torch.cuda.synchronize()
        for j in range(ndst):
            got = from_dev(dsts[j], np.uint8)
            assert same(got[dos[j]:dos[j] + size], src_h[so:so + size]), (so, ndst, j, dos[j])
            assert (got[:dos[j]] == 0xAB).all() and (got[dos[j] + size:] == 0xAB).all(), (so, ndst, j, dos[j])


def test_copy_fanout_several_sources_in_one_call(L):
    """The copies of an all-gather inside a cluster of four: every member's block goes to all
    four receive buffers, the member's own included; 4 sources x 4 destinations in one call,
    then 20 sources x 3 (more than one launch's worth).  A destination equal to its source is
    skipped; empty copies are nothing."""
    import torch
    m, blk = 4, 70001
    hs = [rand_bytes(blk, 900 + r) for r in range(m)]
    recv = [torch.full((m * blk + 32,), 0x5A, dtype=torch.uint8, device="cuda") for _ in range(m)]
    for r in range(m):                                          # in place: member r's block already sits at r * blk
        recv[r][r * blk:(r + 1) * blk] = to_dev(hs[r])
    torch.cuda.synchronize()
    L.copy_fanout([(recv[r].data_ptr() + r * blk, [recv[h].data_ptr() + r * blk for h in range(m)], blk) for r in range(m)]
                  + [(recv[0].data_ptr(), [], blk), (recv[0].data_ptr(), [recv[1].data_ptr()], 0)])
    torch.cuda.synchronize()
    want = np.concatenate(hs)
    for h in range(m):
        got = from_dev(recv[h], np.uint8)
        assert same(got[:m * blk], want), h
        assert (got[m * blk:] == 0x5A).all(), h
    ns, nd, size = 20, 3, 5000
    srcs_h = [rand_bytes(size, 1000 + i) for i in range(ns)]
    srcs = [to_dev(h) for h in srcs_h]
    outs = [[torch.full((size + 16,), 0x77, dtype=torch.uint8, device="cuda") for _ in range(nd)] for _ in range(ns)]
    L.copy_fanout([(srcs[i].data_ptr(), [o.data_ptr() for o in outs[i]], size) for i in range(ns)])
    torch.cuda.synchronize()
    for i in range(ns):
        for o in outs[i]:
            got = from_dev(o, np.uint8)
            assert same(got[:size], srcs_h[i]) and (got[size:] == 0x77).all(), i


def test_copy_fanout_beyond_4GiB_offsets(L):
    """A block that straddles the 4 GiB mark of its buffers (descriptors are per tile, offsets 64-bit)."""
    import torch
    big = (1 << 32) + (1 << 20)
    src = torch.empty(big, dtype=torch.uint8, device="cuda")
    dsts = [torch.empty(big, dtype=torch.uint8, device="cuda") for _ in range(2)]
    at, n = (1 << 32) - 300_000, 600_000
    h = rand_bytes(n, 4)
    src[at:at + n] = to_dev(h)
    for d in dsts:
        d[at - 16:at + n + 16] = 0x3C
    torch.cuda.synchronize()
    L.copy_fanout([(src.data_ptr() + at, [d.data_ptr() + at for d in dsts], n)])
    torch.cuda.synchronize()
    for d in dsts:
        got = from_dev(d[at - 16:at + n + 16], np.uint8)
        assert same(got[16:16 + n], h) and (got[:16] == 0x3C).all() and (got[16 + n:] == 0x3C).all()


def test_device_async_store_and_bounded_load(L):
    """deviceAsyncStore sets the flag, deviceAsyncLoad returns once it is set; with
    the flag never set the load gives up after its spin bound and exits normally."""
    import torch
    flag = torch.zeros(4, dtype=torch.uint8, device="cuda")
    st = L.current_stream()
    lib = L.lib()
    lib.deviceAsyncStore(C.byref(st), flag.data_ptr())
    lib.deviceAsyncLoad(C.byref(st), flag.data_ptr())      # already set: no spinning
    torch.cuda.synchronize()
    assert flag.cpu().tolist() == [1, 0, 0, 0]
    lib.flagcxLocalSetMaxSpinCount(8)                      # host-forced tiny bound
    try:
        lib.deviceAsyncLoad(C.byref(st), flag.data_ptr() + 1)  # never set
        torch.cuda.synchronize()
    finally:
        lib.flagcxLocalSetMaxSpinCount(-1)
    assert flag.cpu().tolist() == [1, 0, 0, 0]


def test_device_fifo_producer_host_consumer(L):
    """One lane enqueues Send, Recv, Term, Wait into the pinned FIFO; the host
    dequeues them in order; the kernel's final wait ends once the queue is drained."""
    import time
    import torch
    lib = L.lib()
    fifo = C.c_void_p()
    assert lib.flagcxLocalFifoInit(C.byref(fifo)) == 0
    words = (C.c_uint64 * 3).from_address(fifo.value)
    assert list(words) == [16, 0, 0]
    empty = L.DeviceTrigger(1, 1)
    assert lib.flagcxLocalFifoDequeue(fifo, C.byref(empty)) == 0 and (empty.fst, empty.snd) == (0, 0)
    send = torch.zeros(1000, dtype=torch.float32, device="cuda")
    recv = torch.zeros(1000, dtype=torch.float32, device="cuda")
    lib.flagcxLocalSetMaxSpinCount(1 << 22)          # seconds, not minutes, if the host stalls
    try:
        st = L.current_stream()
        assert lib.flagcxLocalP2pDemo(send.data_ptr(), recv.data_ptr(), 1000, int(L.DataType.Float32), 3, 5,
                                      fifo, C.byref(st)) == 0
        got = []
        deadline = time.time() + 20
        while len(got) < 4 and time.time() < deadline:
            t = L.DeviceTrigger()
            assert lib.flagcxLocalFifoDequeue(fifo, C.byref(t)) == 0
            if words[1] > len(got):                  # consumed advanced: a real entry
                got.append((t.addr, t.count, t.peer, t.datatype, t.prim))
        torch.cuda.synchronize()
    finally:
        lib.flagcxLocalSetMaxSpinCount(-1)
    f32 = int(L.DataType.Float32)
    assert got == [(send.data_ptr(), 1000, 3, f32, 0), (recv.data_ptr(), 1000, 5, f32, 1),
                   (0, 0, 0, 0, 2), (0, 0, 0, 0, 3)]
    assert list(words) == [16, 4, 4]
    assert lib.flagcxLocalFifoDestroy(fifo) == 0


def test_device_fifo_full_queue_gives_up(L):
    """Nobody dequeues and the queue is pre-filled: the producer's bounded wait
    expires and the kernel exits without writing."""
    import torch
    lib = L.lib()
    fifo = C.c_void_p()
    assert lib.flagcxLocalFifoInit(C.byref(fifo)) == 0
    words = (C.c_uint64 * 3).from_address(fifo.value)
    words[2] = 16                                    # produced - consumed == capacity
    lib.flagcxLocalSetMaxSpinCount(4)
    try:
        st = L.current_stream()
        assert lib.flagcxLocalP2pDemo(1 << 20, 1 << 21, 8, 7, 0, 1, fifo, C.byref(st)) == 0
        torch.cuda.synchronize()
    finally:
        lib.flagcxLocalSetMaxSpinCount(-1)
    assert list(words) == [16, 0, 16]
    assert lib.flagcxLocalFifoDestroy(fifo) == 0
