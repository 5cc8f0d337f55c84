"""Seeded random cases through every way into the reduce (one call, a batch, a gated batch opened descriptor by
descriptor, the resident queue) against the CPU oracle: random element type, operation, number of inputs, length,
and positions of the buffers inside their 128-byte cache lines (all equal modulo 16 where the entry point asks for
it, anything element-aligned otherwise).  Bit equality, any NaN payload where the arithmetic gives NaN, and guard
elements before and after every output untouched."""
import random

import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import dev_empty, from_dev, is_float, make_inputs, same, to_dev

pytestmark = pytest.mark.gpu

DTS = [O.INT8, O.UINT8, O.INT32, O.UINT32, O.INT64, O.UINT64, O.FP16, O.FP32, O.FP64, O.BF16]
OPS = [O.SUM, O.PROD, O.MAX, O.MIN, O.AVG]


@pytest.fixture(scope="module")
def L():
    import torch
    assert torch.cuda.is_available()
    from flagcx_amd import local
    assert local.lib().flagcxLocalInit() == 0
    local.lib().flagcxLocalSetMaxSpinCount(1 << 21)
    yield local
    local.lib().flagcxLocalSetMaxSpinCount(-1)


def one_case(L, rnd, mode, side, large):
    import torch
    dt, op = rnd.choice(DTS), rnd.choice(OPS)
    isz = np.dtype(O.NP_OF[dt]).itemsize
    k = rnd.randint(1, 10) if mode == "reduce" else rnd.randint(1, 8)
    nd = 1 if mode == "reduce" else rnd.randint(1, 5)
    line, gran = 128 // isz, 16 // isz
    keep, descs = [], []
    for _ in range(nd):
        n = rnd.randint(100_000, 2_000_000) if large else rnd.choice([1, 3, 17, 255, 1024, 4097, rnd.randint(1, 60_000)])
        pad = 256 // isz
        ins = make_inputs(dt, k, n + pad, seed=rnd.randint(0, 1 << 30), op=op)
        same16 = mode != "reduce" or rnd.random() < 0.6
        base = rnd.randrange(0, line) if rnd.random() < 0.7 else 0
        if same16:   # every buffer at the same offset modulo 16 bytes, possibly on different 16-byte granules of its line
            offs = [base + gran * rnd.randrange(0, 4) if rnd.random() < 0.5 else base for _ in range(k)]
            do = base + gran * rnd.randrange(0, 4) if rnd.random() < 0.5 else base
        else:
            offs = [rnd.randrange(0, line) for _ in range(k)]
            do = rnd.randrange(0, line)
        devs = [to_dev(a) for a in ins]
        out = dev_empty(n + pad, isz, fill=0)
        keep.append((ins, out, offs, do, n))
        descs.append(([devs[j].data_ptr() + offs[j] * isz for j in range(k)], out.data_ptr() + do * isz, n, devs))
    torch.cuda.synchronize()
    plain = [d[:3] for d in descs]
    if mode == "reduce":
        srcs, dst, n = plain[0]
        L.check(L.lib().flagcxLocalReduce(L._ptr_array(srcs), k, dst, n, int(dt), int(op), L._sref(L.current_stream())))
    elif mode == "batch":
        L.reduce_batch(plain, op, dt, k)
    elif mode == "gated":
        with L.Gate() as gate:
            with torch.cuda.stream(side):
                first = gate.reduce_batch(plain, op, dt, k)
            for i in range(nd):
                gate.open(first + i + 1)
            side.synchronize()
            assert gate.query()[2] == 0
    else:
        q = L.ReduceFifo(8, 8, dt, op)
        try:
            with q:
                ticket = 0
                for srcs, dst, n in plain:
                    ticket = q.enqueue_reduce(srcs, dst, n)
                q.wait(ticket)
        finally:
            q.close()
    torch.cuda.synchronize()
    for ins, out, offs, do, n in keep:
        rc, want = O.reduce([np.ascontiguousarray(ins[j][offs[j]:offs[j] + n]) for j in range(k)], dt, op)
        got = from_dev(out, ins[0].dtype)
        nan = is_float(dt) and op in (O.SUM, O.PROD, O.AVG)
        what = (mode, dt, op, k, offs, do, n)
        assert rc == 0 and same(got[do:do + n], want, nan_class=nan, dtype=dt), what
        assert not got[:do].tobytes().strip(b"\0") and not got[do + n:].tobytes().strip(b"\0"), what


@pytest.mark.parametrize("mode", ["reduce", "batch", "gated", "queue"])
def test_random_cases_match_the_oracle(L, mode):
    import torch
    rnd = random.Random({"reduce": 11, "batch": 12, "gated": 13, "queue": 14}[mode])
    side = torch.cuda.Stream()
    for i in range(120 if mode != "queue" else 40):
        one_case(L, rnd, mode, side, large=False)
    for i in range(12 if mode != "queue" else 6):
        one_case(L, rnd, mode, side, large=True)


SPECIAL = {
    O.FP16: (np.uint16, [0x0000, 0x8000, 0x7c00, 0xfc00, 0x7e00, 0xfe01, 0x7c01, 0x0001, 0x8001, 0x03ff, 0x0400, 0x7bff,
                         0xfbff, 0x3c00, 0xbc00, 0x3555, 0x4248]),
    O.BF16: (np.uint16, [0x0000, 0x8000, 0x7f80, 0xff80, 0x7fc0, 0xffc1, 0x7f81, 0x0001, 0x8001, 0x007f, 0x0080, 0x7f7f,
                         0xff7f, 0x3f80, 0xbf80, 0x3eab, 0x4049]),
    O.FP32: (np.uint32, [0x00000000, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0xffc00001, 0x7f800001, 0x00000001,
                         0x80000001, 0x007fffff, 0x00800000, 0x7f7fffff, 0xff7fffff, 0x3f800000, 0xbf800000, 0x3eaaaaab,
                         0x40490fdb]),
    O.FP64: (np.uint64, [0x0, 0x8000000000000000, 0x7ff0000000000000, 0xfff0000000000000, 0x7ff8000000000000,
                         0xfff8000000000001, 0x7ff0000000000001, 0x1, 0x8000000000000001, 0x000fffffffffffff,
                         0x0010000000000000, 0x7fefffffffffffff, 0xffefffffffffffff, 0x3ff0000000000000,
                         0xbff0000000000000, 0x3fd5555555555555, 0x400921fb54442d18]),
}


@pytest.mark.parametrize("mode", ["reduce", "batch", "gated", "queue"])
def test_random_special_values_match_the_oracle(L, mode):
    """Inputs drawn from NaNs with payloads, infinities, signed zeros, denormals and the extremes of each
    floating-point type: min and max return the chosen input bit for bit (the last NaN or zero wins as in the
    reference's templates), sums and products give the oracle's bits or a NaN where it gives a NaN."""
    import torch
    rnd = random.Random({"reduce": 31, "batch": 32, "gated": 33, "queue": 34}[mode])
    side = torch.cuda.Stream()
    for case in range(150 if mode != "queue" else 60):
        dt, op = rnd.choice(list(SPECIAL)), rnd.choice(OPS)
        ut, pool = SPECIAL[dt]
        npdt = np.dtype(O.NP_OF[dt])
        isz = npdt.itemsize
        k = rnd.randint(1, 8)
        n = rnd.choice([1, 9, 100, 1031, rnd.randint(1, 20_000)])
        rng = np.random.default_rng(rnd.randint(0, 1 << 30))
        ins = [np.array(pool, dtype=ut)[rng.integers(0, len(pool), n + 32)].view(npdt) for _ in range(k)]
        off = rnd.randrange(0, 16)
        devs = [to_dev(a) for a in ins]
        out = dev_empty(n + 32, isz, fill=0)
        srcs = [d.data_ptr() + off * isz for d in devs]
        dst = out.data_ptr() + off * isz
        torch.cuda.synchronize()
        if mode == "reduce":
            L.check(L.lib().flagcxLocalReduce(L._ptr_array(srcs), k, dst, n, int(dt), int(op), L._sref(L.current_stream())))
        elif mode == "batch":
            h = n // 2
            L.reduce_batch([(srcs, dst, h), ([p + h * isz for p in srcs], dst + h * isz, n - h)] if h else [(srcs, dst, n)],
                           op, dt, k)
        elif mode == "gated":
            with L.Gate() as gate:
                with torch.cuda.stream(side):
                    gate.reduce_batch([(srcs, dst, n)], op, dt, k)
                gate.open(1)
                side.synchronize()
                assert gate.query()[2] == 0
        else:
            q = L.ReduceFifo(4, 8, dt, op)
            try:
                with q:
                    q.wait(q.enqueue_reduce(srcs, dst, n))
            finally:
                q.close()
        torch.cuda.synchronize()
        rc, want = O.reduce([np.ascontiguousarray(a[off:off + n]) for a in ins], dt, op)
        got = from_dev(out, npdt)[off:off + n]
        assert rc == 0 and same(got, want, nan_class=op in (O.SUM, O.PROD, O.AVG), dtype=dt), (mode, case, dt, op, k, n, off)
