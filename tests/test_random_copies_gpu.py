"""Seeded random cases through the byte movers (copy, memset, strided pack / unpack, pointer-list pack / unpack)
against numpy: random sizes, and random positions of source and destination inside their 128-byte cache lines.
Exact bytes, and guard bytes around every destination untouched."""
import random

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def L():
    import torch
    assert torch.cuda.is_available()
    from flagcx_amd import local
    assert local.lib().flagcxLocalInit() == 0
    return local


def size_of(rnd, large):
    if large:
        return rnd.randint(1 << 20, 6 << 20)
    return rnd.choice([1, 2, 15, 16, 17, 127, 128, 1023, 1024, 1025, 4096, rnd.randint(1, 200_000)])


def check(got, want, lo, n, what):
    assert np.array_equal(got[lo:lo + n], want), what
    assert (got[:lo] == 0x5A).all() and (got[lo + n:] == 0x5A).all(), what


@pytest.mark.parametrize("large", [False, True], ids=["small", "large"])
def test_random_copies_match_numpy(L, large):
    import torch
    rnd = random.Random(21 if large else 22)
    g = np.random.default_rng(5)
    for case in range(16 if large else 150):
        kind = rnd.choice(["memcpy", "memset", "pack", "unpack", "pack_list", "unpack_list"])
        so, do = rnd.randrange(0, 128), rnd.randrange(0, 128)
        if kind == "memcpy":
            n = size_of(rnd, large)
            h = g.integers(0, 256, n + 256, dtype=np.uint8)
            src = torch.from_numpy(h).cuda()
            dst = torch.full((n + 384,), 0x5A, dtype=torch.uint8, device="cuda")
            L.memcpy(dst.data_ptr() + do, src.data_ptr() + so, n)
            torch.cuda.synchronize()
            check(dst.cpu().numpy(), h[so:so + n], do, n, (kind, so, do, n))
        elif kind == "memset":
            n, v = size_of(rnd, large), rnd.randrange(0, 256)
            dst = torch.full((n + 384,), 0x5A, dtype=torch.uint8, device="cuda")
            L.memset(dst.data_ptr() + do, v, n)
            torch.cuda.synchronize()
            check(dst.cpu().numpy(), np.full(n, v, np.uint8), do, n, (kind, do, n, v))
        else:
            nch = rnd.randint(1, 9)
            cb = size_of(rnd, large) // (nch if large else 1) + 1
            if kind in ("pack", "unpack"):
                stride = cb + rnd.choice([0, 1, 16, 100, cb])
                sparse = g.integers(0, 256, so + stride * nch + 256, dtype=np.uint8)
                chunks = np.concatenate([sparse[so + i * stride:so + i * stride + cb] for i in range(nch)])
                if kind == "pack":
                    src = torch.from_numpy(sparse).cuda()
                    dst = torch.full((nch * cb + 384,), 0x5A, dtype=torch.uint8, device="cuda")
                    L.pack(dst.data_ptr() + do, src.data_ptr() + so, nch, cb, stride)
                    torch.cuda.synchronize()
                    check(dst.cpu().numpy(), chunks, do, nch * cb, (kind, so, do, nch, cb, stride))
                else:
                    packed = torch.from_numpy(np.concatenate([np.zeros(so, np.uint8), chunks])).cuda()
                    dst = torch.full((do + stride * nch + 384,), 0x5A, dtype=torch.uint8, device="cuda")
                    L.unpack(dst.data_ptr() + do, packed.data_ptr() + so, nch, cb, stride)
                    torch.cuda.synchronize()
                    got = dst.cpu().numpy()
                    want = np.full(got.shape, 0x5A, np.uint8)
                    for i in range(nch):
                        want[do + i * stride:do + i * stride + cb] = chunks[i * cb:(i + 1) * cb]
                    assert np.array_equal(got, want), (kind, so, do, nch, cb, stride)
            else:
                offs = [rnd.randrange(0, 128) for _ in range(nch)]
                hosts = [g.integers(0, 256, cb + 256, dtype=np.uint8) for _ in range(nch)]
                chunks = np.concatenate([hosts[i][offs[i]:offs[i] + cb] for i in range(nch)])
                if kind == "pack_list":
                    srcs = [torch.from_numpy(h).cuda() for h in hosts]
                    dst = torch.full((nch * cb + 384,), 0x5A, dtype=torch.uint8, device="cuda")
                    L.pack_list(dst.data_ptr() + do, [s.data_ptr() + offs[i] for i, s in enumerate(srcs)], cb)
                    torch.cuda.synchronize()
                    check(dst.cpu().numpy(), chunks, do, nch * cb, (kind, offs, do, nch, cb))
                else:
                    packed = torch.from_numpy(np.concatenate([np.zeros(so, np.uint8), chunks])).cuda()
                    dsts = [torch.full((cb + 384,), 0x5A, dtype=torch.uint8, device="cuda") for _ in range(nch)]
                    L.unpack_list([d.data_ptr() + offs[i] for i, d in enumerate(dsts)], packed.data_ptr() + so, cb)
                    torch.cuda.synchronize()
                    for i, d in enumerate(dsts):
                        check(d.cpu().numpy(), chunks[i * cb:(i + 1) * cb], offs[i], cb, (kind, offs, so, nch, cb, i))


@pytest.mark.parametrize("large", [False, True], ids=["small", "large"])
def test_random_fanout_copies_match_numpy(L, large):
    """flagcxLocalCopyFanout: 1..5 copies per call, each one source to 1..12 destinations, random sizes and
    random positions inside the cache lines (mostly at the source's offset modulo 16, which shares one read
    of the source; the rest go as plain copies), now and then a destination that is the source itself."""
    import torch
    rnd = random.Random(41 if large else 42)
    g = np.random.default_rng(6)
    for case in range(10 if large else 120):
        copies, keep = [], []
        for _ in range(rnd.randint(1, 5)):
            n = size_of(rnd, large)
            so = rnd.randrange(0, 128)
            h = g.integers(0, 256, n + 256, dtype=np.uint8)
            src = torch.from_numpy(h).cuda()
            outs = []
            for j in range(rnd.randint(1, 12)):
                do = (so % 16) + 16 * rnd.randrange(0, 8) if rnd.random() < 0.8 else rnd.randrange(0, 128)
                outs.append((torch.full((n + 384,), 0x5A, dtype=torch.uint8, device="cuda"), do))
            ptrs = [o.data_ptr() + do for o, do in outs]
            if rnd.random() < 0.2:
                ptrs.insert(rnd.randrange(0, len(ptrs) + 1), src.data_ptr() + so)      # in place: skipped
            copies.append((src.data_ptr() + so, ptrs, n))
            keep.append((h, so, n, outs, src))
        L.copy_fanout(copies)
        torch.cuda.synchronize()
        for h, so, n, outs, src in keep:
            assert np.array_equal(src.cpu().numpy(), h), (case, "source changed")
            for o, do in outs:
                check(o.cpu().numpy(), h[so:so + n], do, n, (case, so, do, n, len(outs)))
