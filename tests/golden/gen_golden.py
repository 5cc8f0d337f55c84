"""Writes tests/golden/ref_reduce_vectors.npz: seeded inputs and the outputs of the
reference's OWN sum<T>/min<T>/max<T> templates (flagcx/service/utils.h:681-709),
reached through oracle/_ref/libflagcx_ref.so (built by `make -C oracle` from the
reference tree where it lies).  Run in the build container only:

    python tests/golden/gen_golden.py

The fixture holds data only (inputs and expected outputs).  Folds are done the way
the reference's ring does them: res = OP(op1 = next input, op2 = res)
(flagcx/service/bootstrap.cc:651-653); the reduce-scatter cases use the ring's
order r = rank+1, ..., rank (mod nranks) (bootstrap.cc:597-598).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import cpu_oracle as O  # noqa: E402

N = 523           # odd: exercises vector tails
K = 8
NAMES = {O.INT8: "i8", O.UINT8: "u8", O.INT32: "i32", O.UINT32: "u32", O.INT64: "i64",
         O.UINT64: "u64", O.FP32: "f32", O.FP64: "f64"}
OPN = {O.SUM: "sum", O.MAX: "max", O.MIN: "min"}


def make_inputs(dt, rng, safe):
    npdt = np.dtype(O.NP_OF[dt])
    if npdt.kind == "f":
        x = rng.uniform(-1, 1, size=(K, N)).astype(npdt)
        if not safe:
            fi = np.finfo(npdt)
            sp = np.array([0.0, -0.0, np.inf, -np.inf, np.nan, fi.tiny, -fi.tiny,
                           fi.smallest_subnormal, -fi.smallest_subnormal, fi.max, -fi.max,
                           1.0, -1.0, fi.eps, 1.0 + fi.eps, 3.0], dtype=npdt)
            # every ordered pair of specials meets in rows (0,1); other rows cycle
            m = len(sp)
            for j in range(K):
                for i in range(m * m):
                    a, b = divmod(i, m)
                    x[j, i] = sp[a] if j % 2 == 0 else sp[(b + j // 2) % m]
        return x
    ii = np.iinfo(npdt)
    if safe:  # k-way sums cannot overflow
        lo, hi = ii.min // (2 * K), ii.max // (2 * K)
        return rng.integers(lo, hi, size=(K, N), dtype=npdt, endpoint=True)
    x = rng.integers(ii.min, ii.max, size=(K, N), dtype=npdt, endpoint=True)
    sp = np.array([ii.min, ii.max, 0, 1, ii.max - 1, ii.min + 1], dtype=npdt)
    m = len(sp)
    for j in range(K):
        for i in range(m * m):
            a, b = divmod(i, m)
            x[j, i] = sp[a] if j % 2 == 0 else sp[(b + j // 2) % m]
    return x


def main():
    assert O.ref_lib() is not None, "build oracle/_ref first (make -C oracle)"
    rng = np.random.default_rng(20251125)
    out = {}
    for dt, nm in NAMES.items():
        signed = np.dtype(O.NP_OF[dt]).kind == "i"
        full = make_inputs(dt, rng, safe=False)
        out[f"in_full_{nm}"] = full
        if signed:
            safe = make_inputs(dt, rng, safe=True)
            out[f"in_safe_{nm}"] = safe
        for op, on in OPN.items():
            src = safe if (signed and op == O.SUM) else full
            for k in (2, 3, 8):
                rc, res = O.ref_fold([np.ascontiguousarray(src[j]) for j in range(k)], dt, op)
                assert rc == 0
                out[f"fold_{nm}_{on}_k{k}"] = res
            # equal-block ring reduce-scatter, 4 ranks x 129 elements
            nr, rcount = 4, 129
            for rank in range(nr):
                order = [(rank + 1 + j) % nr for j in range(nr)]
                sl = [np.ascontiguousarray(src[r, rank * rcount:(rank + 1) * rcount]) for r in order]
                rc, res = O.ref_fold(sl, dt, op)
                assert rc == 0
                out[f"ringrs_{nm}_{on}_r{rank}"] = res
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "ref_reduce_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
