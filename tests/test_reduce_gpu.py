"""GPU parity of the N-way reduce (through the C ABI) against the CPU oracle and
the golden vectors made with the reference's own templates.

Bar: bit-exact for integers, min/max and fp32/fp64 arithmetic in the stated fold
order; for fp16/bf16 sum/prod/avg and for avg the stated tolerance is 1 ulp of the
output type - the tests below demand equality with the oracle, which is stricter.
The only relaxation: where an arithmetic result is NaN, any NaN payload is accepted.
"""
import ctypes as C

import numpy as np
import pytest

from oracle import cpu_oracle as O
from tests.util import (ALL_DTYPES, ALL_OPS, DT_NAME, OP_NAME, dev_empty, from_dev, is_float,
                        make_inputs, same, to_dev)

pytestmark = pytest.mark.gpu

GOLD_NAMES = {O.INT8: "i8", O.UINT8: "u8", O.INT32: "i32", O.UINT32: "u32", O.INT64: "i64",
              O.UINT64: "u64", O.FP32: "f32", O.FP64: "f64"}
GOLD_OPS = {O.SUM: "sum", O.MAX: "max", O.MIN: "min"}


@pytest.fixture(scope="module")
def L():
    import torch
    assert torch.cuda.is_available()
    from flagcx_amd import local
    assert local.lib().flagcxLocalInit() == 0
    return local


def gpu_reduce(L, srcs_np, dtype, op, dst_fill=None):
    import torch
    devs = [to_dev(s) for s in srcs_np]
    out = dev_empty(srcs_np[0].size, srcs_np[0].dtype.itemsize, fill=dst_fill)
    L.reduce(devs, out, op, dtype=dtype)
    torch.cuda.synchronize()
    return from_dev(out, srcs_np[0].dtype)


def arith_nan_ok(dtype, op):
    return is_float(dtype) and op in (O.SUM, O.PROD, O.AVG)


# ------------------------------------------------------------------ golden

@pytest.mark.parametrize("dt", list(GOLD_NAMES), ids=lambda d: DT_NAME[d])
@pytest.mark.parametrize("op", list(GOLD_OPS), ids=lambda o: OP_NAME[o])
def test_reduce_matches_reference_golden(L, golden, dt, op):
    nm, on = GOLD_NAMES[dt], GOLD_OPS[op]
    signed = np.dtype(O.NP_OF[dt]).kind == "i"
    src = golden[f"in_safe_{nm}"] if (signed and op == O.SUM) else golden[f"in_full_{nm}"]
    for k in (2, 3, 8):
        got = gpu_reduce(L, [np.ascontiguousarray(src[j]) for j in range(k)], dt, op)
        assert same(got, golden[f"fold_{nm}_{on}_k{k}"], nan_class=arith_nan_ok(dt, op), dtype=dt), (nm, on, k)


@pytest.mark.parametrize("dt", list(GOLD_NAMES), ids=lambda d: DT_NAME[d])
@pytest.mark.parametrize("op", list(GOLD_OPS), ids=lambda o: OP_NAME[o])
def test_reduce_scatter_matches_reference_golden(L, golden, dt, op):
    import torch
    nm, on = GOLD_NAMES[dt], GOLD_OPS[op]
    signed = np.dtype(O.NP_OF[dt]).kind == "i"
    src = golden[f"in_safe_{nm}"] if (signed and op == O.SUM) else golden[f"in_full_{nm}"]
    nr, rcount = 4, 129
    send = [to_dev(np.ascontiguousarray(src[r, :nr * rcount])) for r in range(nr)]
    for rank in range(nr):
        out = dev_empty(rcount, src.dtype.itemsize)
        L.reduce_scatter(send, rank, out, op, dtype=dt)
        torch.cuda.synchronize()
        assert same(from_dev(out, src.dtype), golden[f"ringrs_{nm}_{on}_r{rank}"],
                    nan_class=arith_nan_ok(dt, op), dtype=dt), (nm, on, rank)


# ------------------------------------------------------- oracle, all types

@pytest.mark.parametrize("dt", ALL_DTYPES, ids=lambda d: DT_NAME[d])
@pytest.mark.parametrize("op", ALL_OPS, ids=lambda o: OP_NAME[o])
def test_reduce_matches_oracle_all_types(L, dt, op):
    # sizes straddle the vector width, one wavefront tile and several tiles
    for k, n in ((1, 5), (2, 1), (2, 4096 + 3), (3, 1000), (4, 70001), (5, 33), (8, 262144 + 17),
                 (9, 5000), (16, 12345), (64, 777)):
        srcs = make_inputs(dt, k, n, seed=1000 * dt + 10 * op + k, op=op)
        rc, want = O.reduce(srcs, dt, op)
        assert rc == 0
        got = gpu_reduce(L, srcs, dt, op)
        assert same(got, want, nan_class=arith_nan_ok(dt, op), dtype=dt), (DT_NAME[dt], OP_NAME[op], k, n)


@pytest.mark.parametrize("dt", [O.FP16, O.BF16, O.FP32], ids=lambda d: DT_NAME[d])
def test_float_special_values(L, dt):
    # every ordered pair of specials, folded with k = 2 and k = 3
    if dt == O.FP32:
        sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1.17549435e-38, 3.4028235e38,
                       -3.4028235e38, 1.0, -1.0, 1.0000001, 3.0, 1e-40, 16777216.0], dtype=np.float32)
    elif dt == O.FP16:
        sp = np.array([0x0000, 0x8000, 0x7c00, 0xfc00, 0x7e00, 0x0001, 0x8001, 0x0400, 0x7bff, 0xfbff,
                       0x3c00, 0xbc00, 0x3c01, 0x4200, 0x03ff, 0x6800], dtype=np.uint16).view(np.float16)
    else:
        sp = np.array([0x0000, 0x8000, 0x7f80, 0xff80, 0x7fc0, 0x0001, 0x8001, 0x0080, 0x7f7f, 0xff7f,
                       0x3f80, 0xbf80, 0x3f81, 0x4040, 0x007f, 0x4b80], dtype=np.uint16)
    m = len(sp)
    a = np.repeat(sp, m)
    b = np.tile(sp, m)
    c = np.roll(b, 5)
    for op in ALL_OPS:
        for srcs in ([a, b], [a, b, c], [c, a, b, a]):
            srcs = [np.ascontiguousarray(s) for s in srcs]
            rc, want = O.reduce(srcs, dt, op)
            got = gpu_reduce(L, srcs, dt, op)
            assert same(got, want, nan_class=arith_nan_ok(dt, op), dtype=dt), (DT_NAME[dt], OP_NAME[op], len(srcs))


def test_reference_pattern_i_mod_10(L):
    # test/unittest/main.cpp:23-48: every rank holds i % 10, sum = nranks * (i % 10)
    n, k = 1 << 20, 8
    x = (np.arange(n) % 10).astype(np.float32)
    got = gpu_reduce(L, [x] * k, O.FP32, O.SUM)
    assert np.array_equal(got, k * x)
    got = gpu_reduce(L, [x] * k, O.FP32, O.AVG)
    assert np.array_equal(got, x)


# ------------------------------------------------------ alignment, aliasing

@pytest.mark.parametrize("dt", [O.INT8, O.BF16, O.FP32, O.FP64], ids=lambda d: DT_NAME[d])
def test_unaligned_and_mixed_offsets(L, dt):
    import torch
    ts = O.type_size(dt)
    n, k = 10007, 3
    srcs = make_inputs(dt, k, n + 64, seed=77 + dt)
    devs = [to_dev(s) for s in srcs]
    for offs, doff in (((1, 1, 1), 1), ((3, 3, 3), 3), ((0, 1, 2), 0), ((5, 5, 5), 2), ((0, 0, 0), 7)):
        out = dev_empty(n + 64, ts, fill=0x55 if ts == 1 else 0x5555)
        guard = from_dev(out, srcs[0].dtype).copy()
        views = [d[o:o + n] for d, o in zip(devs, offs)]
        L.reduce(views, out[doff:doff + n], O.SUM, dtype=dt)
        torch.cuda.synchronize()
        rc, want = O.reduce([np.ascontiguousarray(s[o:o + n]) for s, o in zip(srcs, offs)], dt, O.SUM)
        got = from_dev(out, srcs[0].dtype)
        assert same(got[doff:doff + n], want, nan_class=is_float(dt), dtype=dt), (offs, doff)
        # nothing outside the destination range was written
        assert same(got[:doff], guard[:doff]) and same(got[doff + n:], guard[doff + n:]), (offs, doff)


@pytest.mark.parametrize("dt,k", [(O.BF16, 8), (O.FP32, 2), (O.INT8, 3), (O.FP64, 1), (O.INT32, 5), (O.FP16, 11)],
                         ids=lambda v: str(v))
def test_positions_inside_cache_lines(L, dt, k):
    """Buffers that start anywhere inside a 128-byte line: the first tile is cut short so that
    later tiles start on a line (of most buffers, or of the destination), tiles may be dealt
    out in runs per XCD, and grids are padded to whole rounds; every byte of the result and
    nothing outside it is written, for sizes of less than a tile, a few tiles and many rounds."""
    import torch
    ts = O.type_size(dt)
    per16 = 16 // ts
    pad = 256 // ts
    for n in (per16 * 3 + 1, 1024 // ts * 5 + 3, 1024 // ts * 200 + per16 + 1):
        srcs = make_inputs(dt, k, n + 2 * pad, seed=31 + dt + n % 97)
        devs = [to_dev(s) for s in srcs]
        # (source offsets, destination offset) in elements: all at the same place in their lines,
        # sources on a line and the destination not, the other way round, every source elsewhere
        # (same offset modulo 16 bytes), and sources that need the lane-shift kernel
        cases = [([per16] * k, per16), ([4 * per16] * k, 4 * per16), ([0] * k, per16), ([5 * per16] * k, per16),
                 ([(j % 8) * per16 for j in range(k)], 2 * per16), ([1 + j % 3 for j in range(k)], per16),
                 ([1 + j % 3 for j in range(k)], 3 * per16 + 1)]
        for offs, doff in cases:
            out = dev_empty(n + 2 * pad, ts, fill=0x55 if ts == 1 else 0x5555)
            guard = from_dev(out, srcs[0].dtype).copy()
            views = [d[o:o + n] for d, o in zip(devs, offs)]
            L.reduce(views, out[doff:doff + n], O.SUM, dtype=dt)
            torch.cuda.synchronize()
            rc, want = O.reduce([np.ascontiguousarray(s[o:o + n]) for s, o in zip(srcs, offs)], dt, O.SUM)
            got = from_dev(out, srcs[0].dtype)
            assert same(got[doff:doff + n], want, nan_class=is_float(dt), dtype=dt), (n, offs, doff)
            assert same(got[:doff], guard[:doff]) and same(got[doff + n:], guard[doff + n:]), (n, offs, doff)
        # in place on the first input, inside a line
        o = 3 * per16
        want = O.reduce([np.ascontiguousarray(s[o:o + n]) for s in srcs], dt, O.SUM)[1]
        views = [d[o:o + n] for d in devs]
        L.reduce(views, views[0], O.SUM, dtype=dt)
        torch.cuda.synchronize()
        assert same(from_dev(devs[0], srcs[0].dtype)[o:o + n], want, nan_class=is_float(dt), dtype=dt), n


@pytest.mark.parametrize("dt", [O.FP32, O.BF16, O.INT32], ids=lambda d: DT_NAME[d])
def test_in_place_on_any_input(L, dt):
    import torch
    k, n = 4, 50001
    srcs = make_inputs(dt, k, n, seed=5 + dt)
    rc, want = O.reduce(srcs, dt, O.SUM)
    for j in range(k):
        devs = [to_dev(s) for s in srcs]
        L.reduce(devs, devs[j], O.SUM, dtype=dt)
        torch.cuda.synchronize()
        assert same(from_dev(devs[j], srcs[0].dtype), want, nan_class=is_float(dt), dtype=dt), j


def test_null_stream_blocks_and_launcher_symbol(L):
    import torch
    srcs = make_inputs(O.FP32, 2, 4097, seed=3)
    rc, want = O.reduce(srcs, O.FP32, O.SUM)
    devs = [to_dev(s) for s in srcs]
    out = dev_empty(4097, 4)
    torch.cuda.synchronize()
    L.reduce(devs, out, O.SUM, dtype=O.FP32, stream=None)  # NULL: returns after completion
    assert same(from_dev(out, np.float32), want)
    # the launcher-convention entry: void fn(flagcxStream_t, void *args)
    out2 = dev_empty(4097, 4)
    arr = (C.c_void_p * 2)(devs[0].data_ptr(), devs[1].data_ptr())
    args = L.ReduceArgs(arr, out2.data_ptr(), 4097, 2, O.FP32, O.SUM, -1)
    st = L.current_stream()
    L.lib().flagcxLocalReduceFunc(C.byref(st), C.byref(args))
    torch.cuda.synchronize()
    assert args.result == 0 and same(from_dev(out2, np.float32), want)


# --------------------------------------------------------------- ring forms

@pytest.mark.parametrize("dt,op", [(O.FP32, O.SUM), (O.INT32, O.MAX), (O.FP64, O.MIN), (O.BF16, O.SUM),
                                   (O.FP16, O.AVG), (O.FP32, O.PROD)],
                         ids=lambda v: str(v))
def test_all_reduce_matches_ring_oracle(L, dt, op):
    import torch
    strict = dt in O.REF_DTYPES and op in O.REF_OPS
    ts = O.type_size(dt)
    for nranks, n in ((2, 1000), (3, (9 << 20) // ts + 5), (8, (5 << 20) // ts + 1), (1, 333)):
        send = make_inputs(dt, nranks, n, seed=nranks * 7 + dt, op=op)
        rc, want = O.ring_allreduce(send, dt, op, strict=strict)
        assert rc == 0
        devs = [to_dev(s) for s in send]
        out = dev_empty(n, ts)
        L.all_reduce(devs, out, op, dtype=dt)
        torch.cuda.synchronize()
        assert same(from_dev(out, send[0].dtype), want, nan_class=arith_nan_ok(dt, op), dtype=dt), (nranks, n)
    # in place on rank 1's buffer
    send = make_inputs(dt, 3, 4099, seed=1, op=op)
    rc, want = O.ring_allreduce(send, dt, op, strict=strict)
    devs = [to_dev(s) for s in send]
    L.all_reduce(devs, devs[1], op, dtype=dt)
    torch.cuda.synchronize()
    assert same(from_dev(devs[1], send[0].dtype), want, nan_class=arith_nan_ok(dt, op), dtype=dt)


@pytest.mark.parametrize("dt,op", [(O.FP32, O.SUM), (O.FP16, O.AVG), (O.INT64, O.MIN)], ids=lambda v: str(v))
def test_reduce_scatter_and_chunked_match_oracle(L, dt, op):
    import torch
    strict = dt in O.REF_DTYPES and op in O.REF_OPS
    ts = O.type_size(dt)
    nranks, rcount = 8, 30011
    send = make_inputs(dt, nranks, nranks * rcount, seed=21 + dt, op=op)
    devs = [to_dev(s) for s in send]
    for rank in (0, 3, 7):
        rc, want = O.reduce_scatter_rank(send, rank, rcount, dt, op, strict=strict)
        assert rc == 0
        out = dev_empty(rcount, ts)
        L.reduce_scatter(devs, rank, out, op, dtype=dt)
        out2 = dev_empty(rcount, ts)
        L.reduce_scatter(devs, rank, out2, op, dtype=dt, chunkbytes=4096 * ts)
        torch.cuda.synchronize()
        assert same(from_dev(out, send[0].dtype), want, nan_class=arith_nan_ok(dt, op), dtype=dt), rank
        assert same(from_dev(out2, send[0].dtype), want, nan_class=arith_nan_ok(dt, op), dtype=dt), rank
    # in place: recvbuff == sendbuffs[rank] + rank*recvcount (flagcx.h:356)
    rank = 2
    rc, want = O.reduce_scatter_rank(send, rank, rcount, dt, op, strict=strict)
    L.reduce_scatter(devs, rank, devs[rank][rank * rcount:(rank + 1) * rcount], op, dtype=dt)
    torch.cuda.synchronize()
    got = from_dev(devs[rank], send[0].dtype)[rank * rcount:(rank + 1) * rcount]
    assert same(got, want, nan_class=arith_nan_ok(dt, op), dtype=dt)


def test_reduce_scatter_reference_pattern(L):
    # test/perf/test_reducescatter.cpp:86-97: value floor(i / recvcount) -> shard r = nranks * r
    import torch
    k, rcount = 8, 4096
    x = to_dev((np.arange(k * rcount) // rcount).astype(np.float32))
    for rank in range(k):
        out = dev_empty(rcount, 4)
        L.reduce_scatter([x] * k, rank, out, O.SUM, dtype=O.FP32)
        torch.cuda.synchronize()
        assert np.array_equal(from_dev(out, np.float32), np.full(rcount, k * rank, np.float32))


# ------------------------------------------------------- batch and triggers

@pytest.mark.parametrize("dt,op,k", [(O.BF16, O.SUM, 8), (O.FP32, O.MIN, 3), (O.INT32, O.SUM, 2), (O.FP16, O.AVG, 9)],
                         ids=lambda v: str(v))
def test_reduce_batch_matches_oracle(L, dt, op, k):
    """Many descriptors of different sizes and alignments in one call; each must
    equal its own flagcxLocalReduce / oracle result."""
    import torch
    ts = O.type_size(dt)
    sizes = [1, 7, 4096, 100003, 33, 65536, 12345] * 6      # 42 descriptors -> two launches
    srcs_h, devs, outs, descs = [], [], [], []
    for i, n in enumerate(sizes):
        off = i % 3                                          # some descriptors unaligned
        hs = make_inputs(dt, k, n + 4, seed=900 + i, op=op)
        ds = [to_dev(h) for h in hs]
        out = dev_empty(n + 4, ts, fill=0)
        srcs_h.append([np.ascontiguousarray(h[off:off + n]) for h in hs])
        devs.append(ds)
        outs.append(out)
        descs.append(([d.data_ptr() + off * ts for d in ds], out.data_ptr() + off * ts, n))
    L.reduce_batch(descs, op, dt, k)
    torch.cuda.synchronize()
    for i, n in enumerate(sizes):
        off = i % 3
        rc, want = O.reduce(srcs_h[i], dt, op)
        got = from_dev(outs[i], srcs_h[i][0].dtype)[off:off + n]
        assert same(got, want, nan_class=arith_nan_ok(dt, op), dtype=dt), (i, n)


def test_chunk_pipeline_as_one_batch_equals_chunked(L):
    """The 4 MiB chunks of a reduce-scatter shard as one batch call."""
    import torch
    nranks, rcount, rank = 8, 1 << 20, 5
    chunk = 1 << 16
    send = [to_dev(h) for h in make_inputs(O.FP16, nranks, nranks * rcount, seed=31)]
    ref = dev_empty(rcount, 2)
    L.reduce_scatter(send, rank, ref, O.AVG, dtype=O.FP16)
    out = dev_empty(rcount, 2)
    descs = []
    for c in range(rcount // chunk):
        srcs = [send[(rank + 1 + j) % nranks].data_ptr() + (rank * rcount + c * chunk) * 2 for j in range(nranks)]
        descs.append((srcs, out.data_ptr() + c * chunk * 2, chunk))
    L.reduce_batch(descs, O.AVG, O.FP16, nranks)
    torch.cuda.synchronize()
    assert torch.equal(ref, out)


def test_reduce_triggers_in_order_with_dependencies(L):
    """Binary reduce descriptors in the reference's 256-bit layout, executed in
    order: a ring-style chain where each trigger consumes the previous output."""
    import torch
    n = 50000
    hs = make_inputs(O.FP32, 4, n, seed=8)
    ds = [to_dev(h) for h in hs]
    t1 = dev_empty(n, 4)
    t2 = dev_empty(n, 4)
    t3 = dev_empty(n, 4)
    other = dev_empty(n, 4)
    T = L.ReduceTrigger.make
    f32 = int(L.DataType.Float32)
    trig = [T(ds[1].data_ptr(), ds[0].data_ptr(), t1.data_ptr(), n, f32, O.SUM),     # t1 = x1 + x0
            T(ds[2].data_ptr(), t1.data_ptr(), t2.data_ptr(), n, f32, O.SUM),        # t2 = x2 + t1 (depends)
            T(ds[3].data_ptr(), ds[0].data_ptr(), other.data_ptr(), n, f32, O.MAX),  # independent, other op
            T(ds[3].data_ptr(), t2.data_ptr(), t3.data_ptr(), n, f32, O.SUM)]        # t3 = x3 + t2
    L.reduce_triggers(trig)
    torch.cuda.synchronize()
    rc, want = O.reduce(hs, O.FP32, O.SUM)          # ((x0+x1)+x2)+x3 in the ring's operand order
    assert same(from_dev(t3, np.float32), want)
    rc, wmax = O.binary(O.MAX, O.FP32, hs[3], hs[0])
    assert same(from_dev(other, np.float32), wmax)
    # int32 min through a trigger
    hi = make_inputs(O.INT32, 2, 1001, seed=9)
    di = [to_dev(h) for h in hi]
    oi = dev_empty(1001, 4)
    L.reduce_triggers([T(di[0].data_ptr(), di[1].data_ptr(), oi.data_ptr(), 1001, int(L.DataType.Int32), O.MIN)])
    torch.cuda.synchronize()
    rc, wmin = O.binary(O.MIN, O.INT32, hi[0], hi[1])
    assert same(from_dev(oi, np.int32), wmin)


@pytest.mark.parametrize("dt", [O.FP16, O.BF16, O.FP32, O.FP64], ids=lambda d: DT_NAME[d])
def test_special_values_on_the_generic_and_element_paths(L, dt):
    """NaN / inf / signed zero / subnormal handling must not depend on which kernel
    runs: 9 inputs take the any-k kernel, mismatched alignment the element kernel."""
    import torch
    npdt = np.dtype(O.NP_OF[dt])
    if dt == O.BF16:
        sp = np.array([0x0000, 0x8000, 0x7f80, 0xff80, 0x7fc0, 0x0001, 0x8001, 0x0080, 0x7f7f, 0xff7f,
                       0x3f80, 0xbf80, 0x3f81, 0x4040, 0x007f, 0x4b80], dtype=np.uint16)
    else:
        fi = np.finfo(npdt)
        sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, fi.smallest_subnormal, -fi.smallest_subnormal, fi.tiny,
                       fi.max, -fi.max, 1.0, -1.0, 1.0 + fi.eps, 3.0, fi.tiny / 2, 2.0 ** (fi.nmant + 1)], dtype=npdt)
    m = len(sp)
    rows = [np.ascontiguousarray(np.roll(np.tile(sp, m), 3 * j) if j % 2 else np.repeat(sp, m)) for j in range(9)]
    ts = O.type_size(dt)
    for op in ALL_OPS:
        rc, want = O.reduce(rows, dt, op)
        got = gpu_reduce(L, rows, dt, op)                       # k = 9: any-k kernel
        assert same(got, want, nan_class=arith_nan_ok(dt, op), dtype=dt), (DT_NAME[dt], OP_NAME[op], "k9")
        # k = 3 with one input offset by one element: element kernel
        pads = [np.concatenate([r, r[:4]]) for r in rows[:3]]
        devs = [to_dev(p) for p in pads]
        out = dev_empty(m * m, ts)
        views = [devs[0][1:1 + m * m], devs[1][0:m * m], devs[2][0:m * m]]
        L.reduce(views, out, op, dtype=dt)
        torch.cuda.synchronize()
        rc, want = O.reduce([np.ascontiguousarray(pads[0][1:1 + m * m]), rows[1], rows[2]], dt, op)
        assert same(from_dev(out, npdt), want, nan_class=arith_nan_ok(dt, op), dtype=dt), (DT_NAME[dt], OP_NAME[op], "elem")


def _tie_columns(k, op, want_columns=64):
    """Columns of k fp16 values whose fp32 fold lands on a tie between two fp16 values while the exact result
    does not: rounding the fold's fp32 result (what the fold is defined to do) and rounding the exact result once
    (what an operation fused into the conversion does) give different fp16 values there."""
    rng = np.random.default_rng(1000 + 10 * k + op)
    found = []
    for _ in range(8):   # (such columns are about 6 in 100 000 for products; sums of a few halves are exact in fp32,
                         # and a quotient by 3, 5, 6 or 7 never ends in the bits of a tie)
        if sum(c.shape[1] for c in found) >= want_columns:
            break
        f = rng.standard_normal((k, 1 << 20))
        cand = (1.0 + 0.1 * f if op == O.PROD else f).astype(np.float16)
        acc32 = cand[0].astype(np.float32)
        exact = cand[0].astype(np.float64)
        for j in range(1, k):
            if op == O.PROD:
                acc32 = cand[j].astype(np.float32) * acc32
                exact = cand[j].astype(np.float64) * exact
            else:
                acc32 = cand[j].astype(np.float32) + acc32
                exact = cand[j].astype(np.float64) + exact
        if op == O.AVG:
            acc32 = acc32 / np.float32(k)
            exact = exact / np.float64(k)
        twice, once = acc32.astype(np.float16), exact.astype(np.float16)
        found.append(cand[:, twice.view(np.uint16) != once.view(np.uint16)])
    cols = np.concatenate(found, axis=1)[:, :want_columns]
    assert cols.shape[1] >= 8, "no rounding ties found for this fold"
    return cols


@pytest.mark.parametrize("op,k", [(O.PROD, 3), (O.PROD, 4), (O.PROD, 5), (O.PROD, 6), (O.PROD, 7), (O.PROD, 8)],
                         ids=lambda v: str(v))
def test_fp16_fold_rounds_in_fp32_before_it_rounds_to_fp16(L, op, k):
    """The fold of halves is a chain of fp32 operations, each rounded to fp32, and ONE final conversion.  A
    compiler that fuses the last operation into the conversion rounds the exact result once instead, which
    differs wherever the fp32 result is a tie between two fp16 values (6 elements in 100 000 of random data; it
    happened for products, in the few head and tail elements only, whose loop over the inputs unrolls).  Every
    element here is such a case, through one call, a batch, a gated batch and the queue, head and tail included."""
    import torch
    cols = _tie_columns(k, op)
    n = 4096 + 13
    ins = [np.ascontiguousarray(np.resize(cols[j], n + 16)) for j in range(k)]
    devs = [to_dev(a) for a in ins]
    rc, want = O.reduce([np.ascontiguousarray(a[1:n + 1]) for a in ins], O.FP16, op)
    assert rc == 0
    outs = [dev_empty(n + 16, 2, fill=0) for _ in range(4)]
    srcs = [d.data_ptr() + 2 for d in devs]          # one element in: 7 head elements, a tail
    dst = [o.data_ptr() + 2 for o in outs]
    L.check(L.lib().flagcxLocalReduce(L._ptr_array(srcs), k, dst[0], n, int(O.FP16), int(op),
                                      L._sref(L.current_stream())))
    L.reduce_batch([(srcs, dst[1], n // 2), ([p + (n // 2) * 2 for p in srcs], dst[1] + (n // 2) * 2, n - n // 2)],
                   op, O.FP16, k)
    torch.cuda.synchronize()
    L.lib().flagcxLocalSetMaxSpinCount(1 << 21)
    side = torch.cuda.Stream()
    try:
        with L.Gate() as gate:
            with torch.cuda.stream(side):
                gate.reduce_batch([(srcs, dst[2], n)], op, O.FP16, k)
            gate.open(1)
            side.synchronize()
            assert gate.query()[2] == 0
        q = L.ReduceFifo(4, k, O.FP16, op)
        try:
            with q:
                q.wait(q.enqueue_reduce(srcs, dst[3], n))
        finally:
            q.close()
    finally:
        L.lib().flagcxLocalSetMaxSpinCount(-1)
    torch.cuda.synchronize()
    for name, out in zip(("one call", "batch", "gated batch", "queue"), outs):
        got = from_dev(out, np.float16)[1:n + 1]
        differing = np.nonzero(got.view(np.uint16) != want.view(np.uint16))[0]
        assert differing.size == 0, (name, op, k, differing.size, differing[:8])


# ------------------------------------------- more than eight inputs, batch by batch

@pytest.mark.parametrize("dt", ALL_DTYPES, ids=lambda d: DT_NAME[d])
@pytest.mark.parametrize("op", ALL_OPS, ids=lambda o: OP_NAME[o])
def test_more_than_eight_inputs_every_batch_remainder(L, dt, op):
    """More than eight inputs are folded in batches (eight at a time where every source
    shares the output's address modulo 16, four at a time through lane shifts otherwise):
    every length of the last batch, with the inputs aligned, all at one other offset, and each at an offset of its own."""
    import torch
    ts = O.type_size(dt)
    per16 = 16 // ts
    n = 2 * 1024 // ts * 3 + 37            # a few tiles and a ragged end
    for k in list(range(9, 18)) + [20, 23, 33, 64]:
        srcs = make_inputs(dt, k, n + 64, seed=5000 + 100 * dt + 10 * op + k, op=op)
        devs = [to_dev(s) for s in srcs]
        for name, offs, doff in (("aligned", [0] * k, 0),
                                 ("one offset", [1] * k, 0),
                                 ("mixed", [(3 * j + 1) % (2 * per16) for j in range(k)], per16 // 2 if per16 > 1 else 1)):
            out = dev_empty(n + 64, ts, fill=0x55 if ts == 1 else 0x5555)
            guard = from_dev(out, srcs[0].dtype).copy()
            L.reduce([d[o:o + n] for d, o in zip(devs, offs)], out[doff:doff + n], op, dtype=dt)
            torch.cuda.synchronize()
            rc, want = O.reduce([np.ascontiguousarray(s[o:o + n]) for s, o in zip(srcs, offs)], dt, op)
            assert rc == 0
            got = from_dev(out, srcs[0].dtype)
            assert same(got[doff:doff + n], want, nan_class=arith_nan_ok(dt, op), dtype=dt), (k, name)
            assert same(got[:doff], guard[:doff]) and same(got[doff + n:], guard[doff + n:]), (k, name)


@pytest.mark.parametrize("dt", [O.INT8, O.UINT8], ids=lambda d: DT_NAME[d])
@pytest.mark.parametrize("k", [2, 3, 8, 9, 12])
def test_8bit_folds_on_every_pair_of_byte_values(L, dt, k):
    """8-bit elements are folded four to a 32-bit word with 16-bit packed arithmetic.
    Every pair of byte values, in each of the four positions of a word, against plain
    integer arithmetic done here (not the oracle): sum and product modulo 256, minimum
    and maximum with the type's sign, the average as the wrapped sum divided by k with C
    truncation.  Inputs beyond the first two repeat the second value."""
    npdt = np.dtype(O.NP_OF[dt])
    a = np.repeat(np.arange(256), 256)
    b = np.tile(np.arange(256), 256)
    a = np.concatenate([a, a[:3]])          # 65539 elements: every pair lands in every byte position somewhere
    b = np.concatenate([b, b[:3]])
    a = np.concatenate([np.roll(a, s) for s in range(4)])
    b = np.concatenate([np.roll(b, s) for s in range(4)])
    srcs = [a.astype(np.uint8).view(npdt)] + [b.astype(np.uint8).view(npdt)] * (k - 1)
    av, bv = srcs[0].astype(np.int64), srcs[1].astype(np.int64)

    def wrap(x):
        return (x & 0xFF).astype(np.uint8).view(npdt)

    total = av + (k - 1) * bv
    wrapped_sum = wrap(total).astype(np.int64)
    kk = np.int64(np.array(k).astype(npdt))
    quotient = np.abs(wrapped_sum) // abs(kk) * np.sign(wrapped_sum) * np.sign(kk)   # C division truncates
    prod = av.copy()
    for _ in range(k - 1):
        prod = (prod * bv) & 0xFF
    want = {O.SUM: wrap(total), O.PROD: wrap(prod), O.MAX: np.maximum(av, bv).astype(npdt),
            O.MIN: np.minimum(av, bv).astype(npdt), O.AVG: quotient.astype(npdt)}
    for op in ALL_OPS:
        got = gpu_reduce(L, srcs, dt, op)
        assert same(got, want[op]), (DT_NAME[dt], OP_NAME[op], k)
