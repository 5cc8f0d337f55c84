"""Pins the CPU oracle: against golden vectors made with the reference's own
templates, against those templates live (where oracle/_ref was built), and for
what the reference does not define (fp16/bf16, prod, avg) against numpy / torch
library arithmetic, exact cases and invariants."""
import numpy as np
import pytest
import torch

from oracle import cpu_oracle as O

NAMES = {O.INT8: "i8", O.UINT8: "u8", O.INT32: "i32", O.UINT32: "u32", O.INT64: "i64",
         O.UINT64: "u64", O.FP32: "f32", O.FP64: "f64"}
OPN = {O.SUM: "sum", O.MAX: "max", O.MIN: "min"}


def same(a, b, nan_class=False):
    """Bit equality; with nan_class, NaNs only need to be NaN on both sides."""
    if nan_class and a.dtype.kind == "f":
        na, nb = np.isnan(a), np.isnan(b)
        if not np.array_equal(na, nb):
            return False
        return a[~na].tobytes() == b[~nb].tobytes()
    return a.tobytes() == b.tobytes()


# ------------------------------------------------------------------ golden

@pytest.mark.parametrize("dt", list(NAMES))
@pytest.mark.parametrize("op", list(OPN))
def test_fold_matches_reference_golden(golden, dt, op):
    nm, on = NAMES[dt], OPN[op]
    signed = np.dtype(O.NP_OF[dt]).kind == "i"
    src = golden[f"in_safe_{nm}"] if (signed and op == O.SUM) else golden[f"in_full_{nm}"]
    for k in (2, 3, 8):
        rc, got = O.reduce([np.ascontiguousarray(src[j]) for j in range(k)], dt, op)
        assert rc == 0
        # a sum of two NaNs may keep either payload depending on operand order
        assert same(got, golden[f"fold_{nm}_{on}_k{k}"], nan_class=(op == O.SUM)), (nm, on, k)


@pytest.mark.parametrize("dt", list(NAMES))
@pytest.mark.parametrize("op", list(OPN))
def test_ring_reduce_scatter_matches_reference_golden(golden, dt, op):
    nm, on = NAMES[dt], OPN[op]
    signed = np.dtype(O.NP_OF[dt]).kind == "i"
    src = golden[f"in_safe_{nm}"] if (signed and op == O.SUM) else golden[f"in_full_{nm}"]
    nr, rcount = 4, 129
    send = [np.ascontiguousarray(src[r, :nr * rcount]) for r in range(nr)]
    ts = send[0].dtype.itemsize
    rc, outs = O.ring_reduce_scatter(send, [r * rcount * ts for r in range(nr)],
                                     [rcount * ts] * nr, dt, op, strict=True)
    assert rc == 0
    for rank in range(nr):
        want = golden[f"ringrs_{nm}_{on}_r{rank}"]
        assert same(outs[rank], want, nan_class=(op == O.SUM)), (nm, on, rank)
        rc, one = O.reduce_scatter_rank(send, rank, rcount, dt, op, strict=True)
        assert rc == 0 and same(one, want, nan_class=(op == O.SUM))


# ------------------------------------------------------- live reference

needs_ref = pytest.mark.skipif(O.ref_lib() is None, reason="oracle/_ref not built here")


@needs_ref
@pytest.mark.parametrize("dt", list(NAMES))
@pytest.mark.parametrize("op", list(OPN))
def test_binary_matches_reference_live(dt, op):
    rng = np.random.default_rng(dt * 10 + op)
    npdt = np.dtype(O.NP_OF[dt])
    n = 4099
    if npdt.kind == "f":
        a = rng.standard_normal(n).astype(npdt)
        b = rng.standard_normal(n).astype(npdt)
        b[::7] = a[::7]
    else:
        ii = np.iinfo(npdt)
        lo, hi = (ii.min // 4, ii.max // 4) if op == O.SUM else (ii.min, ii.max)
        a = rng.integers(lo, hi, n, dtype=npdt, endpoint=True)
        b = rng.integers(lo, hi, n, dtype=npdt, endpoint=True)
    rc1, r1 = O.binary(op, dt, a, b, strict=True)
    rc2, r2 = O.ref_binary(op, dt, a, b)
    assert rc1 == rc2 == 0
    assert same(r1, r2)


@needs_ref
def test_reference_rejects_what_strict_rejects():
    a = np.zeros(8, dtype=np.uint16)
    for dt in (O.FP16, O.BF16, 10, 77):
        assert O.ref_binary(O.SUM, dt, a, a)[0] == O.INVALID
        assert O.binary(O.SUM, dt, a, a, strict=True)[0] == O.INVALID
    f = np.zeros(8, dtype=np.float32)
    for op in (O.PROD, O.AVG, 5):
        assert O.ref_binary(op, O.FP32, f, f)[0] == O.INVALID
        assert O.binary(op, O.FP32, f, f, strict=True)[0] == O.INVALID


@needs_ref
def test_enum_values_match_reference_headers():
    R = O.ref_lib()
    want = dict(flagcxSuccess=0, flagcxUnhandledDeviceError=1, flagcxSystemError=2,
                flagcxInternalError=3, flagcxInvalidArgument=4, flagcxInvalidUsage=5,
                flagcxRemoteError=6, flagcxInProgress=7, flagcxUnhandledCCLError=8,
                flagcxNotSupported=9, flagcxInt8=O.INT8, flagcxUint8=O.UINT8,
                flagcxInt32=O.INT32, flagcxUint32=O.UINT32, flagcxInt64=O.INT64,
                flagcxUint64=O.UINT64, flagcxFloat16=O.FP16, flagcxFloat=O.FP32,
                flagcxFloat64=O.FP64, flagcxBfloat16=O.BF16, flagcxSum=O.SUM,
                flagcxProd=O.PROD, flagcxMax=O.MAX, flagcxMin=O.MIN, flagcxAvg=O.AVG)
    for k, v in want.items():
        assert R.ref_enum(k.encode()) == v, k


# ---------------------------------------------------------------- basics

def test_type_sizes():
    # flagcx/flagcx.cc:30-61
    assert [O.type_size(d) for d in range(10)] == [1, 1, 4, 4, 8, 8, 2, 4, 8, 2]
    assert O.type_size(10) == 0 and O.type_size(-1) == 0


def test_fp32_sum_is_sequential_numpy_fold():
    rng = np.random.default_rng(0)
    srcs = [rng.uniform(-1, 1, 10007).astype(np.float32) for _ in range(8)]
    acc = srcs[0].copy()
    for s in srcs[1:]:
        acc = s + acc
    rc, got = O.reduce(srcs, O.FP32, O.SUM)
    assert rc == 0 and same(got, acc)
    # and the order matters: a different order gives different bits somewhere
    rc, rev = O.reduce(srcs[::-1], O.FP32, O.SUM)
    assert not same(rev, acc)


def test_single_rank_is_copy():
    x = np.arange(100, dtype=np.int32)
    for op in (O.SUM, O.PROD, O.MAX, O.MIN, O.AVG):
        rc, got = O.reduce([x], O.INT32, op)
        assert rc == 0 and same(got, x)
    rc, got = O.ring_allreduce([x], O.INT32, O.SUM, strict=True)
    assert rc == 0 and same(got, x)


def test_minmax_argument_order_signed_zero_and_nan():
    # std::min(a,b) = (b<a)?b:a ; std::max(a,b) = (a<b)?b:a  with a = op1
    pz, nz, nan = np.float32(0.0), np.float32(-0.0), np.float32(np.nan)
    a = np.array([pz, nz, nan, 1.0, nan], dtype=np.float32)
    b = np.array([nz, pz, 1.0, nan, nan], dtype=np.float32)
    for op in (O.MIN, O.MAX):
        rc, r = O.binary(op, O.FP32, a, b, strict=True)
        # ties and unordered keep op1
        assert same(r, a)
    # fold: acc = OP(new, acc): the last input wins ties, and only its NaN survives
    rc, r = O.reduce([b, a], O.FP32, O.MIN)
    assert same(r, a)
    rc, r = O.reduce([a, b], O.FP32, O.MIN)
    assert same(r, b)


def test_integer_sum_wraps():
    a = np.array([127, -128, 100], dtype=np.int8)
    b = np.array([1, -1, 100], dtype=np.int8)
    rc, r = O.binary(O.SUM, O.INT8, a, b, strict=True)
    assert r.tolist() == [-128, 127, -56]
    a = np.array([2**31 - 1], dtype=np.int32)
    rc, r = O.reduce([a, a, a], O.INT32, O.SUM)
    assert r.tolist() == [((3 * (2**31 - 1)) + 2**31) % 2**32 - 2**31]


# ------------------------------------------------------ half conversions

def test_half_to_float_exhaustive_vs_numpy():
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = O.half_to_float(bits)
    # signalling NaNs are quietened on the way through Python floats
    assert same(got, want, nan_class=True)


def test_bf16_to_float_exhaustive_vs_torch():
    bits = np.arange(65536, dtype=np.uint16)
    t = torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    got = O.bf16_to_float(bits)
    assert same(got, t, nan_class=True)


def _probe_floats():
    rng = np.random.default_rng(5)
    xs = [rng.standard_normal(20000).astype(np.float32),
          (rng.standard_normal(20000) * 1e-6).astype(np.float32),
          (rng.standard_normal(5000) * 7e4).astype(np.float32),
          rng.integers(0, 2**32, 40000, dtype=np.uint64).astype(np.uint32).view(np.float32)]
    # every fp16 value, its midpoints to the next value and one ulp(fp32) either side
    h = np.arange(0x7c00, dtype=np.uint16).view(np.float16).astype(np.float64)
    mid = (h[:-1] + h[1:]) / 2
    m32 = mid.astype(np.float32)
    xs += [m32, np.nextafter(m32, np.float32(np.inf)), np.nextafter(m32, np.float32(-np.inf)),
           -m32, np.array([65504, 65519.99, 65520, 65536, 1e30, 2**-24, 2**-25,
                           np.nextafter(np.float32(2**-25), np.float32(1)), 2**-26, 0.0, -0.0,
                           np.inf, -np.inf], dtype=np.float32)]
    x = np.concatenate(xs)
    return x[~np.isnan(x)]


def test_float_to_half_vs_numpy():
    x = _probe_floats()
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = O.float_to_half(x)
    assert same(got, want)
    assert np.isnan(np.array(O.float_to_half([np.nan]), dtype=np.uint16).view(np.float16))[0]


def test_float_to_bf16_vs_torch():
    x = _probe_floats()
    # plus exact ties of the bf16 grid
    b = np.arange(0, 0x7f80, 3, dtype=np.uint32) << 16
    ties = (b | 0x8000).view(np.float32)
    x = np.concatenate([x, ties, -ties, np.nextafter(ties, np.float32(np.inf))])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = O.float_to_bf16(x)
    assert same(got, want)
    nb = O.float_to_bf16([np.nan])[0]
    assert (nb & 0x7f80) == 0x7f80 and (nb & 0x7f) != 0


# --------------------------------------------- half / prod / avg semantics

@pytest.mark.parametrize("k", [2, 3, 8])
def test_fp16_sum_vs_numpy_fp32_fold(k):
    rng = np.random.default_rng(k)
    srcs = [rng.standard_normal(5003).astype(np.float16) for _ in range(k)]
    acc = srcs[0].astype(np.float32)
    for s in srcs[1:]:
        acc = s.astype(np.float32) + acc
    rc, got = O.reduce(srcs, O.FP16, O.SUM)
    assert rc == 0 and same(got, acc.astype(np.float16))
    rc, avg = O.reduce(srcs, O.FP16, O.AVG)
    assert same(avg, (acc / np.float32(k)).astype(np.float16))
    pacc = srcs[0].astype(np.float32)
    for s in srcs[1:]:
        pacc = s.astype(np.float32) * pacc
    rc, prod = O.reduce(srcs, O.FP16, O.PROD)
    assert same(prod, pacc.astype(np.float16))


@pytest.mark.parametrize("k", [2, 5, 8])
def test_bf16_sum_vs_torch_fp32_fold(k):
    g = torch.Generator().manual_seed(k)
    ts = [torch.randn(5003, generator=g).to(torch.bfloat16) for _ in range(k)]
    acc = ts[0].float()
    for t in ts[1:]:
        acc = t.float() + acc
    want = acc.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    srcs = [t.view(torch.int16).numpy().view(np.uint16).copy() for t in ts]
    rc, got = O.reduce(srcs, O.BF16, O.SUM)
    assert rc == 0 and same(got, want)
    want_avg = (acc / k).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    rc, got = O.reduce(srcs, O.BF16, O.AVG)
    assert same(got, want_avg)


def test_half_k2_sum_is_one_correctly_rounded_add():
    # for k = 2 the fp32 sum of two fp16 values is exact, so the result must be the
    # correctly rounded fp16 sum: compare with float64 arithmetic rounded once
    rng = np.random.default_rng(9)
    a = rng.standard_normal(20000).astype(np.float16)
    b = (rng.standard_normal(20000) * 3).astype(np.float16)
    want = (a.astype(np.float64) + b.astype(np.float64)).astype(np.float16)
    rc, got = O.reduce([a, b], O.FP16, O.SUM)
    assert same(got, want)


def test_half_minmax_returns_input_bits():
    #             +0      -0      nan     1       -inf    +inf
    pat = {O.FP16: (0x0000, 0x8000, 0x7e01, 0x3c00, 0xfc00, 0x7c00),
           O.BF16: (0x0000, 0x8000, 0x7fc1, 0x3f80, 0xff80, 0x7f80)}
    for dt, (pz, nz, nan, one, ninf, pinf) in pat.items():
        a = np.array([pz, nz, nan, one, ninf], dtype=np.uint16)
        b = np.array([nz, pz, one, nan, pinf], dtype=np.uint16)
        rc, r = O.binary(O.MIN, dt, a, b)
        assert rc == 0 and r.tolist() == [pz, nz, nan, one, ninf]
        rc, r = O.binary(O.MAX, dt, a, b)
        assert rc == 0 and r.tolist() == [pz, nz, nan, one, pinf]


@pytest.mark.parametrize("dt", [O.INT32, O.UINT8, O.INT64, O.FP32, O.FP64, O.FP16, O.BF16])
def test_small_integer_patterns_are_exact(dt):
    # the reference's own test pattern: i % 10 on every rank, sum = nranks * (i % 10)
    # (test/unittest/main.cpp:23-48)
    n, k = 1000, 8
    vals = (np.arange(n) % 10)
    if dt == O.BF16:
        enc = lambda v: torch.tensor(v, dtype=torch.float32).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16).copy()
        dec = lambda a: torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16).float().numpy()
    else:
        enc = lambda v: np.asarray(v).astype(O.NP_OF[dt])
        dec = lambda a: a.astype(np.float64)
    srcs = [enc(vals) for _ in range(k)]
    rc, s = O.reduce(srcs, dt, O.SUM)
    assert rc == 0 and np.array_equal(dec(s), k * vals)
    rc, a = O.reduce(srcs, dt, O.AVG)
    assert np.array_equal(dec(a), vals)
    rc, m = O.reduce(srcs, dt, O.MAX)
    assert np.array_equal(dec(m), vals)
    small = [enc(np.arange(n) % 3 + 1) for _ in range(3)]
    rc, p = O.reduce(small, dt, O.PROD)
    assert np.array_equal(dec(p), (np.arange(n) % 3 + 1) ** 3)


def test_avg_fp32_is_sum_then_division():
    rng = np.random.default_rng(3)
    for k in (2, 3, 7, 8):
        srcs = [rng.standard_normal(3001).astype(np.float32) for _ in range(k)]
        acc = srcs[0].copy()
        for s in srcs[1:]:
            acc = s + acc
        rc, got = O.reduce(srcs, O.FP32, O.AVG)
        assert same(got, acc / np.float32(k))
    ints = [np.array([7, -7, 9], dtype=np.int32)] * 2 + [np.array([1, -1, 0], dtype=np.int32)]
    rc, got = O.reduce(ints, O.INT32, O.AVG)
    assert got.tolist() == [5, -5, 6]  # C division truncates toward zero


# ------------------------------------------------------------ ring logic

def test_chunk_table_closed_forms():
    M = 1 << 20
    # C1: 64 MiB over 2 ranks -> 2 x 32 MiB (bootstrap.cc:719-738)
    assert O.ring_chunk_table(64 * M, 4, 2) == ([0, 32 * M], [32 * M, 32 * M])
    # below nranks * 4 MiB the tail ranks get nothing and offset == size
    assert O.ring_chunk_table(1024, 4, 4) == ([0, 1024, 1024, 1024], [1024, 0, 0, 0])
    assert O.ring_chunk_table(9 * M, 4, 4) == ([0, 4 * M, 8 * M, 9 * M], [4 * M, 4 * M, M, 0])
    # chunk rounded up to the element size
    off, ln = O.ring_chunk_table(8 * 5 * M + 8, 8, 3)
    assert off[1] % 8 == 0 and sum(ln) == 8 * 5 * M + 8
    for size in (0, 1, 4 * M, 4 * M + 1, 33 * M + 7):
        for n in (1, 2, 3, 8):
            for ts in (1, 2, 4, 8):
                sz = size // ts * ts
                off, ln = O.ring_chunk_table(sz, ts, n)
                assert sum(ln) == sz
                pos = 0
                for o, l in zip(off, ln):
                    assert o == (pos if l else sz)
                    pos += l
                chunk = max(-(-sz // n), 4 * M)
                chunk = -(-chunk // ts) * ts
                assert max(ln) == min(chunk, sz)


@pytest.mark.parametrize("nranks", [2, 3, 4, 8])
def test_ring_allreduce_reference_pattern(nranks):
    # i % 10 on every rank -> nranks * (i % 10); spans >1 chunk so the table matters
    n = (9 << 20) // 4 + 13
    x = (np.arange(n) % 10).astype(np.float32)
    rc, out = O.ring_allreduce([x.copy() for _ in range(nranks)], O.FP32, O.SUM, strict=True)
    assert rc == 0 and np.array_equal(out, nranks * x)


def test_reduce_scatter_reference_pattern():
    # test/perf/test_reducescatter.cpp:86-97: value floor(i / recvcount) -> shard r = k*r
    k, rcount = 8, 1000
    x = (np.arange(k * rcount) // rcount).astype(np.float32)
    for rank in range(k):
        rc, out = O.reduce_scatter_rank([x] * k, rank, rcount, O.FP32, O.SUM, strict=True)
        assert rc == 0 and np.array_equal(out, np.full(rcount, k * rank, np.float32))


def test_ring_order_is_rotation_ending_at_own_rank():
    # With min over signed zeros, std::min keeps op1 = the local chunk, so chunk c
    # ends with rank c's own zero; with NaNs, only rank c's NaN survives.
    k, rcount = 4, 5
    send = []
    for r in range(k):
        v = np.zeros(k * rcount, dtype=np.float32)
        if r % 2:
            v = -v
        send.append(v)
    send[2][0:rcount] = np.nan          # rank 2's NaN in chunk 0: dropped
    send[1][rcount:2 * rcount] = np.nan  # rank 1's NaN in chunk 1: survives
    for rank in range(k):
        rc, out = O.reduce_scatter_rank(send, rank, rcount, O.FP32, O.MIN, strict=True)
        want = send[rank][rank * rcount:(rank + 1) * rcount]
        assert rc == 0 and same(out, want), rank


def test_ring_equals_fold_over_rotation_fp32():
    rng = np.random.default_rng(11)
    k, rcount = 5, 777
    send = [rng.uniform(-1, 1, k * rcount).astype(np.float32) for _ in range(k)]
    for rank in range(k):
        rc, out = O.reduce_scatter_rank(send, rank, rcount, O.FP32, O.SUM, strict=True)
        sl = [send[(rank + 1 + j) % k][rank * rcount:(rank + 1) * rcount].copy() for j in range(k)]
        acc = sl[0]
        for s in sl[1:]:
            acc = s + acc
        assert same(out, acc)
        # the non-strict path (used for the extensions) takes the same order
        rc, out2 = O.reduce_scatter_rank(send, rank, rcount, O.FP32, O.AVG)
        assert same(out2, acc / np.float32(k))


def test_strict_ring_rejects_extensions():
    h = [np.zeros(16, dtype=np.float16)] * 2
    assert O.ring_allreduce(h, O.FP16, O.SUM, strict=True)[0] == O.INVALID
    f = [np.zeros(16, dtype=np.float32)] * 2
    assert O.ring_allreduce(f, O.FP32, O.AVG, strict=True)[0] == O.INVALID
    assert O.ring_allreduce(f, O.FP32, O.AVG, strict=False)[0] == 0


# ----------------------------------------------------------- byte movers

def test_refresh_ranges():
    for op, zeroes in ((O.SUM, True), (O.MAX, False), (O.MIN, False)):
        buf = np.arange(1, 101, dtype=np.float32)
        O.refresh(buf, 10, 20, 30, 80, op)  # region [10,90): keep [30,60)
        want = np.arange(1, 101, dtype=np.float32)
        if zeroes:
            want[10:30] = 0
            want[60:90] = 0
        assert same(buf, want)


def test_pack_unpack_round_trip():
    rng = np.random.default_rng(2)
    nch, cb, stride = 8, 100, 800
    src = rng.integers(0, 256, nch * stride, dtype=np.uint8)
    packed = O.pack(src, nch, cb, stride)
    want = src.reshape(nch, stride)[:, :cb].reshape(-1)
    assert same(packed, want)
    dst = np.full(nch * stride, 0xEE, dtype=np.uint8)
    O.unpack(dst, packed, nch, cb, stride)
    d2 = dst.reshape(nch, stride)
    assert same(np.ascontiguousarray(d2[:, :cb]).reshape(-1), want)
    assert (d2[:, cb:] == 0xEE).all()
