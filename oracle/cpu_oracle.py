"""ctypes loader for the CPU oracle (oracle/flagcx_oracle.c) and, where it was
built, the library around the reference's own templates (oracle/_ref).

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py.  The product package never imports this module.

Arrays are numpy; bf16 data is carried as uint16 bit patterns with dtype code 9.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

# flagcx/include/flagcx.h:27-44
INT8, UINT8, INT32, UINT32, INT64, UINT64, FP16, FP32, FP64, BF16 = range(10)
# flagcx/include/flagcx.h:47-57
SUM, PROD, MAX, MIN, AVG = range(5)
INVALID = 4

NP_OF = {INT8: np.int8, UINT8: np.uint8, INT32: np.int32, UINT32: np.uint32,
         INT64: np.int64, UINT64: np.uint64, FP16: np.float16, FP32: np.float32,
         FP64: np.float64, BF16: np.uint16}
REF_DTYPES = (INT8, UINT8, INT32, UINT32, INT64, UINT64, FP32, FP64)
REF_OPS = (SUM, MAX, MIN)

_lib = None
_ref = None


def build():
    subprocess.run(["make", "-C", HERE], check=True, capture_output=True)


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(HERE, "libflagcx_oracle.so")
        if not os.path.exists(path):
            build()
        L = C.CDLL(path)
        vp, sz, i = C.c_void_p, C.c_size_t, C.c_int
        L.oracle_type_size.restype = sz
        L.oracle_type_size.argtypes = [i]
        L.oracle_binary.argtypes = [i, i, vp, vp, vp, sz, i]
        L.oracle_reduce.argtypes = [C.POINTER(vp), i, vp, sz, i, i]
        L.oracle_ring_reduce_scatter.argtypes = [C.POINTER(vp), C.POINTER(vp), i,
                                                 C.POINTER(sz), C.POINTER(sz), i, i, i]
        L.oracle_ring_chunk_table.argtypes = [sz, sz, i, C.POINTER(sz), C.POINTER(sz)]
        L.oracle_ring_chunk_table.restype = None
        L.oracle_ring_allreduce.argtypes = [C.POINTER(vp), vp, i, sz, i, i, i]
        L.oracle_reduce_scatter_rank.argtypes = [C.POINTER(vp), vp, i, i, sz, i, i, i]
        L.oracle_refresh.argtypes = [vp, sz, sz, sz, sz, sz, i]
        L.oracle_refresh.restype = None
        L.oracle_pack.argtypes = [vp, vp, sz, sz, sz]
        L.oracle_pack.restype = None
        L.oracle_unpack.argtypes = [vp, vp, sz, sz, sz]
        L.oracle_unpack.restype = None
        L.oracle_half_to_float.argtypes = [C.c_uint16]
        L.oracle_half_to_float.restype = C.c_float
        L.oracle_float_to_half.argtypes = [C.c_float]
        L.oracle_float_to_half.restype = C.c_uint16
        L.oracle_bf16_to_float.argtypes = [C.c_uint16]
        L.oracle_bf16_to_float.restype = C.c_float
        L.oracle_float_to_bf16.argtypes = [C.c_float]
        L.oracle_float_to_bf16.restype = C.c_uint16
        L.oracle_time_reduce.argtypes = [C.POINTER(vp), i, vp, sz, i, i, i, i, i]
        L.oracle_time_reduce.restype = C.c_double
        _lib = L
    return _lib


def ref_lib():
    """The reference's own sum/min/max templates, or None when not built."""
    global _ref
    if _ref is None:
        path = os.path.join(HERE, "_ref", "libflagcx_ref.so")
        if not os.path.exists(path):
            return None
        L = C.CDLL(path)
        L.ref_binary.argtypes = [C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t]
        L.ref_enum.argtypes = [C.c_char_p]
        L.ref_adaptor_layout.argtypes = [C.POINTER(C.c_size_t), C.c_int]
        _ref = L
    return _ref


def ref_adaptor_layout():
    """sizeof / member offsets of the reference's struct flagcxDeviceAdaptor."""
    out = (C.c_size_t * 64)()
    n = ref_lib().ref_adaptor_layout(out, 64)
    return list(out[:n])


def _ptr(a):
    return C.c_void_p(a.ctypes.data)


def _ptrs(arrs):
    return (C.c_void_p * len(arrs))(*[a.ctypes.data for a in arrs])


def _check(arrs, dtype):
    want = NP_OF.get(dtype)
    for a in arrs:
        assert a.flags["C_CONTIGUOUS"]
        if want is not None:  # same width is enough: uint16 may carry fp16 bits
            assert a.dtype.itemsize == np.dtype(want).itemsize, (a.dtype, want)


def type_size(dtype):
    return lib().oracle_type_size(dtype)


def binary(op, dtype, a, b, strict=False):
    """OP(op1=a, op2=b) -> (rc, result)."""
    _check([a, b], dtype)
    res = np.empty_like(a)
    rc = lib().oracle_binary(op, dtype, _ptr(res), _ptr(a), _ptr(b), a.size, int(strict))
    return rc, res


def ref_binary(op, dtype, a, b):
    """Same through the reference's templates -> (rc, result)."""
    res = np.empty_like(a)
    rc = ref_lib().ref_binary(op, dtype, _ptr(res), _ptr(a), _ptr(b), a.size)
    return rc, res


def reduce(srcs, dtype, op):
    """N-way fold in list order -> (rc, result)."""
    _check(srcs, dtype)
    dst = np.empty_like(srcs[0])
    rc = lib().oracle_reduce(_ptrs(srcs), len(srcs), _ptr(dst), srcs[0].size, dtype, op)
    return rc, dst


def ref_fold(srcs, dtype, op):
    """The fold of reduce() done with the reference's templates: (k-1) passes of
    res = OP(op1=srcs[j], op2=res) as at flagcx/service/bootstrap.cc:651-653."""
    acc = srcs[0].copy()
    for s in srcs[1:]:
        rc = ref_lib().ref_binary(op, dtype, _ptr(acc), _ptr(s), _ptr(acc), acc.size)
        if rc:
            return rc, None
    return 0, acc


def ring_chunk_table(size_bytes, tsize, nranks):
    off = (C.c_size_t * nranks)()
    ln = (C.c_size_t * nranks)()
    lib().oracle_ring_chunk_table(size_bytes, tsize, nranks, off, ln)
    return list(off), list(ln)


def ring_reduce_scatter(sendbuffs, offsets, lengths, dtype, op, strict=False):
    """All ranks of bootstrapRingReduceScatter -> (rc, [recvbuff per rank])."""
    n = len(sendbuffs)
    _check(sendbuffs, dtype)
    ts = max(type_size(dtype), 1)
    outs = [np.zeros(lengths[r] // ts, dtype=sendbuffs[0].dtype) for r in range(n)]
    # zero-length arrays still need a valid pointer
    keep = [o if o.size else np.zeros(1, dtype=o.dtype) for o in outs]
    off = (C.c_size_t * n)(*offsets)
    ln = (C.c_size_t * n)(*lengths)
    rc = lib().oracle_ring_reduce_scatter(_ptrs(sendbuffs), _ptrs(keep), n, off, ln,
                                          dtype, op, int(strict))
    return rc, outs


def ring_allreduce(sendbuffs, dtype, op, strict=False):
    _check(sendbuffs, dtype)
    out = np.empty_like(sendbuffs[0])
    rc = lib().oracle_ring_allreduce(_ptrs(sendbuffs), _ptr(out), len(sendbuffs),
                                     sendbuffs[0].size, dtype, op, int(strict))
    return rc, out


def reduce_scatter_rank(sendbuffs, rank, recvcount, dtype, op, strict=False):
    _check(sendbuffs, dtype)
    out = np.empty(recvcount, dtype=sendbuffs[0].dtype)
    rc = lib().oracle_reduce_scatter_rank(_ptrs(sendbuffs), _ptr(out), len(sendbuffs), rank,
                                          recvcount, dtype, op, int(strict))
    return rc, out


def refresh(buff, start, offset, count, total, op):
    lib().oracle_refresh(_ptr(buff), start, offset, count, total, buff.dtype.itemsize, op)


def pack(src_bytes, nchunks, chunkbytes, srcstride):
    dst = np.empty(nchunks * chunkbytes, dtype=np.uint8)
    lib().oracle_pack(_ptr(dst), _ptr(src_bytes), nchunks, chunkbytes, srcstride)
    return dst


def unpack(dst_bytes, src_bytes, nchunks, chunkbytes, dststride):
    lib().oracle_unpack(_ptr(dst_bytes), _ptr(src_bytes), nchunks, chunkbytes, dststride)


def half_to_float(bits):
    return np.array([lib().oracle_half_to_float(int(b)) for b in bits], dtype=np.float32)


def float_to_half(vals):
    return np.array([lib().oracle_float_to_half(float(v)) for v in vals], dtype=np.uint16)


def bf16_to_float(bits):
    return np.array([lib().oracle_bf16_to_float(int(b)) for b in bits], dtype=np.float32)


def float_to_bf16(vals):
    return np.array([lib().oracle_float_to_bf16(C.c_float(v)) for v in vals], dtype=np.uint16)


def time_reduce(srcs, dst, dtype, op, nthreads=1, warmup=1, iters=3):
    """Median seconds per N-way reduce on `nthreads` host threads."""
    return lib().oracle_time_reduce(_ptrs(srcs), len(srcs), _ptr(dst), srcs[0].size, dtype, op,
                                    nthreads, warmup, iters)
