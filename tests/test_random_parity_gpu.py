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
