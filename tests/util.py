"""Helpers shared by the GPU parity tests: numpy <-> device tensors by bit pattern,
seeded inputs, comparisons."""
import numpy as np

from oracle import cpu_oracle as O

ALL_DTYPES = list(range(10))
ALL_OPS = [O.SUM, O.PROD, O.MAX, O.MIN, O.AVG]
DT_NAME = {O.INT8: "int8", O.UINT8: "uint8", O.INT32: "int32", O.UINT32: "uint32", O.INT64: "int64",
           O.UINT64: "uint64", O.FP16: "fp16", O.FP32: "fp32", O.FP64: "fp64", O.BF16: "bf16"}
OP_NAME = {O.SUM: "sum", O.PROD: "prod", O.MAX: "max", O.MIN: "min", O.AVG: "avg"}


def same(a, b, nan_class=False, dtype=None):
    """Bit equality.  nan_class: positions where both sides are NaN count as equal
    whatever the payload (dtype tells how to read uint16 carriers)."""
    a = np.ascontiguousarray(a)
    b = np.ascontiguousarray(b)
    if a.shape != b.shape:
        return False
    if not nan_class:
        return a.tobytes() == b.tobytes()
    na, nb = isnan_bits(a, dtype), isnan_bits(b, dtype)
    if not np.array_equal(na, nb):
        return False
    return a[~na].tobytes() == b[~nb].tobytes()


def isnan_bits(a, dtype):
    if dtype == O.BF16:
        u = a.view(np.uint16)
        return ((u & 0x7f80) == 0x7f80) & ((u & 0x7f) != 0)
    if dtype == O.FP16:
        return np.isnan(a.view(np.float16))
    if a.dtype.kind == "f":
        return np.isnan(a)
    return np.zeros(a.shape, dtype=bool)


def is_float(dtype):
    return dtype in (O.FP16, O.FP32, O.FP64, O.BF16)


def f32_to_bf16_bits(x):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (numpy, finite inputs)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = (u + 0x7fff + ((u >> 16) & 1)) >> 16
    return r.astype(np.uint16)


def make_inputs(dtype, k, n, seed, op=O.SUM, dist="normal"):
    """k seeded host arrays of n elements in the numpy carrier type of dtype."""
    rng = np.random.default_rng(seed)
    npdt = np.dtype(O.NP_OF[dtype])
    out = []
    for _ in range(k):
        if dtype == O.BF16:
            f = rng.standard_normal(n).astype(np.float32)
            if op == O.PROD:
                f = (1.0 + 0.1 * f).astype(np.float32)
            out.append(f32_to_bf16_bits(f))
        elif npdt.kind == "f":
            f = rng.standard_normal(n) if dist == "normal" else rng.uniform(-1, 1, n)
            if op == O.PROD:
                f = 1.0 + 0.1 * f
            out.append(f.astype(npdt))
        else:
            ii = np.iinfo(npdt)
            out.append(rng.integers(ii.min, ii.max, n, dtype=npdt, endpoint=True))
    return out


_TORCH_CARRIER = {1: "uint8", 2: "int16", 4: "int32", 8: "int64"}


def to_dev(a, device="cuda"):
    """Upload a numpy array bit for bit as an integer carrier tensor."""
    import torch
    a = np.ascontiguousarray(a)
    carrier = np.dtype(_TORCH_CARRIER[a.dtype.itemsize])
    return torch.from_numpy(a.view(carrier).copy()).to(device)


def dev_empty(n, itemsize, device="cuda", fill=None):
    import torch
    dt = getattr(torch, _TORCH_CARRIER[itemsize])
    if fill is None:
        return torch.empty(n, dtype=dt, device=device)
    return torch.full((n,), fill, dtype=dt, device=device)


def from_dev(t, npdtype):
    return t.cpu().numpy().view(npdtype)
