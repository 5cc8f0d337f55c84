"""ctypes binding of libflagcx_amd.so (include/flagcx_amd.h).

Device memory and streams come from torch; nothing here computes.  Every call
goes through the C ABI, and a missing library is an error (ImportError-like
RuntimeError), never a silent fallback.
"""
import ctypes as C
import enum
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(HERE, "lib", "libflagcx_amd.so")
_lib = None

MAX_RANKS = 64
CHUNKSIZE = 4 * 1024 * 1024


class Result(enum.IntEnum):          # flagcx/include/flagcx.h:12-24
    Success = 0
    UnhandledDeviceError = 1
    SystemError = 2
    InternalError = 3
    InvalidArgument = 4
    InvalidUsage = 5
    RemoteError = 6
    InProgress = 7
    UnhandledCCLError = 8
    NotSupported = 9


class DataType(enum.IntEnum):        # flagcx/include/flagcx.h:27-44
    Int8 = 0
    Uint8 = 1
    Int32 = 2
    Uint32 = 3
    Int64 = 4
    Uint64 = 5
    Float16 = 6
    Float32 = 7
    Float64 = 8
    Bfloat16 = 9


class RedOp(enum.IntEnum):           # flagcx/include/flagcx.h:47-57
    Sum = 0
    Prod = 1
    Max = 2
    Min = 3
    Avg = 4


class FlagcxError(RuntimeError):
    def __init__(self, code, msg):
        super().__init__("flagcx result %d (%s): %s" % (code, Result(code).name if 0 <= code < 10 else "?", msg))
        self.code = code


class Stream(C.Structure):
    """struct flagcxStream { hipStream_t base; } (flagcx/adaptor/include/amd_adaptor.h:14-16)"""
    _fields_ = [("base", C.c_void_p)]


class ReduceArgs(C.Structure):       # flagcxLocalReduceArgs
    _fields_ = [("sendbuffs", C.POINTER(C.c_void_p)), ("recvbuff", C.c_void_p), ("count", C.c_uint64),
                ("nranks", C.c_int32), ("datatype", C.c_int32), ("op", C.c_int32), ("result", C.c_int32)]


class ReduceDesc(C.Structure):       # flagcxLocalReduceDesc
    _fields_ = [("sendbuffs", C.POINTER(C.c_void_p)), ("recvbuff", C.c_void_p), ("count", C.c_size_t)]


class FanoutDesc(C.Structure):       # flagcxLocalFanoutDesc
    _fields_ = [("src", C.c_void_p), ("dsts", C.POINTER(C.c_void_p)), ("ndsts", C.c_int), ("bytes", C.c_size_t)]


class ReduceTrigger(C.Structure):    # flagcxLocalReduceTrigger, 16-byte aligned
    _fields_ = [("value", C.c_uint64 * 4)]
    _pack_ = 16

    @classmethod
    def make(cls, addr1, addr2, addr3, count, datatype, redop, nthreads=0):
        t = cls()
        t.value[0], t.value[1], t.value[2] = addr1, addr2, addr3
        t.value[3] = (count & 0xffffffff) | ((nthreads & 0xffff) << 32) | ((int(datatype) & 0xf) << 48) | \
                     ((int(redop) & 0xf) << 52)
        return t


class DeviceTrigger(C.Structure):    # flagcxLocalDeviceTrigger
    _fields_ = [("fst", C.c_uint64), ("snd", C.c_uint64)]

    @property
    def addr(self):
        return self.fst

    @property
    def count(self):
        return self.snd & 0xffffffff

    @property
    def peer(self):
        return (self.snd >> 32) & 0xfffff

    @property
    def datatype(self):
        return (self.snd >> 52) & 0xf

    @property
    def prim(self):
        return (self.snd >> 56) & 0xf


class CopyArgs(C.Structure):         # flagcxLocalCopyArgs
    _fields_ = [("dst", C.c_void_p), ("src", C.c_void_p), ("size", C.c_uint64), ("result", C.c_int32),
                ("reserved", C.c_int32)]


EXPORTS = [
    "flagcxLocalGetDataTypeSize", "flagcxLocalInit", "flagcxLocalGetErrorString", "flagcxLocalGetLastError",
    "flagcxLocalTune", "flagcxLocalGetTune", "flagcxLocalTuneLoads", "flagcxLocalGetTuneLoads", "flagcxLocalPlaceBuffers", "flagcxLocalReduce", "flagcxLocalReduceScatter", "flagcxLocalReduceScatterChunked",
    "flagcxLocalAllReduce", "flagcxLocalRingChunkTable", "flagcxLocalMemcpy", "flagcxLocalMemset",
    "flagcxLocalRefresh", "flagcxLocalPack", "flagcxLocalUnpack", "flagcxLocalPackList",
    "flagcxLocalUnpackList", "flagcxLocalCopyFanout", "flagcxLocalReduceFunc", "flagcxLocalCopyFunc",
    "flagcxLocalSetMaxSpinCount", "deviceAsyncStore", "deviceAsyncLoad",
    "flagcxLocalReduceBatch", "flagcxLocalReduceBatchSparse", "flagcxLocalReduceTriggers",
    "flagcxLocalGateCreate", "flagcxLocalGateDestroy", "flagcxLocalReduceBatchGated", "flagcxLocalGateOpen",
    "flagcxLocalGateQuery", "flagcxLocalGateOwnStream",
    "flagcxLocalFifoInit", "flagcxLocalFifoDestroy", "flagcxLocalFifoDequeue", "flagcxLocalP2pDemo",
    "flagcxLocalRingCreate", "flagcxLocalRingDestroy", "flagcxLocalRingSendRecv",
    "flagcxLocalRingReduceScatter",
    "flagcxLocalGetDeviceAdaptor", "flagcxLocalDeviceAdaptorLayout",
    "flagcxLocalPlanCreate", "flagcxLocalPlanDestroy", "flagcxLocalPlanImportXml", "flagcxLocalPlanExportXml",
    "flagcxLocalPlanSetAlgorithm", "flagcxLocalPlanSetFused", "flagcxLocalPlanGetTraffic", "flagcxLocalPlanSetChunks", "flagcxLocalPlanSetAlltoAllv", "flagcxLocalPlanExecute", "flagcxLocalPlanGetLastError",
    "flagcxLocalReduceFifoCreate", "flagcxLocalReduceFifoDestroy", "flagcxLocalReduceFifoStart",
    "flagcxLocalReduceFifoStop", "flagcxLocalReduceFifoEnqueue", "flagcxLocalReduceFifoEnqueueReduce",
    "flagcxLocalReduceFifoQuery", "flagcxLocalReduceFifoWait", "flagcxLocalReduceFifoGetGrid",
    "flagcxLocalReduceFifoSetWaves", "flagcxLocalReduceFifoSetLinger", "flagcxLocalReduceFifoSetOwnQueue", "flagcxLocalReduceFifoSetWindow", "flagcxLocalReduceFifoGetType", "flagcxLocalRingReduceScatterFifo",
    "flagcxLocalReduceFifoGetLastError", "flagcxLocalStagedReduceScatterNoAlloc",
]


def lib_path():
    return _LIB_PATH


def lib():
    """The loaded C library; raises if it was not built (python -m flagcx_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            raise RuntimeError("%s is missing: build it with `python -m flagcx_amd.build` "
                               "(there is no fallback implementation)" % _LIB_PATH)
        # PyTorch ships its own copy of the HIP runtime.  Whichever copy a process loads first serves both,
        # and PyTorch does not find its GPUs through another one: where torch is in the process, let it
        # load and initialise its runtime before this library brings in the system's (torch may be imported
        # later by the same process: tests, bench.py and every user of this binding hold their buffers in it).
        try:
            import torch
            torch.cuda.is_available()
        except Exception:
            pass
        L = C.CDLL(_LIB_PATH)
        vp, sz, i, pp = C.c_void_p, C.c_size_t, C.c_int, C.POINTER(C.c_void_p)
        sp = C.POINTER(Stream)
        L.flagcxLocalGetDataTypeSize.restype = sz
        L.flagcxLocalGetDataTypeSize.argtypes = [i]
        L.flagcxLocalInit.argtypes = []
        L.flagcxLocalGetErrorString.restype = C.c_char_p
        L.flagcxLocalGetErrorString.argtypes = [i]
        L.flagcxLocalGetLastError.restype = C.c_char_p
        L.flagcxLocalTune.argtypes = [i, i]
        L.flagcxLocalPlaceBuffers.argtypes = [vp, sz, sz, i, pp]
        L.flagcxLocalGetTune.argtypes = [i, C.POINTER(i)]
        L.flagcxLocalTuneLoads.argtypes = [i, i]
        L.flagcxLocalGetTuneLoads.argtypes = [i, C.POINTER(i)]
        L.flagcxLocalReduce.argtypes = [pp, i, vp, sz, i, i, sp]
        L.flagcxLocalReduceScatter.argtypes = [pp, i, i, vp, sz, i, i, sp]
        L.flagcxLocalReduceScatterChunked.argtypes = [pp, i, i, vp, sz, i, i, sz, sp]
        L.flagcxLocalAllReduce.argtypes = [pp, i, vp, sz, i, i, sp]
        L.flagcxLocalRingChunkTable.argtypes = [sz, i, i, C.POINTER(sz), C.POINTER(sz)]
        L.flagcxLocalMemcpy.argtypes = [vp, vp, sz, sp]
        L.flagcxLocalMemset.argtypes = [vp, i, sz, sp]
        L.flagcxLocalRefresh.argtypes = [vp, sz, sz, sz, sz, i, i, sp]
        L.flagcxLocalPack.argtypes = [vp, vp, sz, sz, sz, sp]
        L.flagcxLocalUnpack.argtypes = [vp, vp, sz, sz, sz, sp]
        L.flagcxLocalPackList.argtypes = [vp, pp, i, sz, sp]
        L.flagcxLocalUnpackList.argtypes = [pp, vp, i, sz, sp]
        L.flagcxLocalCopyFanout.argtypes = [C.POINTER(FanoutDesc), i, sp]
        L.flagcxLocalReduceFunc.restype = None
        L.flagcxLocalReduceFunc.argtypes = [sp, C.POINTER(ReduceArgs)]
        L.flagcxLocalCopyFunc.restype = None
        L.flagcxLocalCopyFunc.argtypes = [sp, C.POINTER(CopyArgs)]
        L.flagcxLocalReduceBatch.argtypes = [C.POINTER(ReduceDesc), i, i, i, i, sp]
        L.flagcxLocalReduceBatchSparse.argtypes = [C.POINTER(ReduceDesc), i, i, i, i, i, sp]
        L.flagcxLocalReduceTriggers.argtypes = [C.POINTER(ReduceTrigger), i, sp]
        L.flagcxLocalFifoInit.argtypes = [C.POINTER(vp)]
        L.flagcxLocalFifoDestroy.argtypes = [vp]
        L.flagcxLocalFifoDequeue.argtypes = [vp, C.POINTER(DeviceTrigger)]
        L.flagcxLocalP2pDemo.argtypes = [vp, vp, sz, i, i, i, vp, sp]
        L.flagcxLocalRingCreate.argtypes = [C.POINTER(vp), vp, sz, i, sz, i]
        L.flagcxLocalRingDestroy.argtypes = [vp]
        L.flagcxLocalRingSendRecv.argtypes = [vp, vp, vp, sz, sp, sp]
        L.flagcxLocalRingReduceScatter.argtypes = [vp, pp, i, i, vp, sz, i, i, sp, sp]
        L.flagcxLocalStagedReduceScatterNoAlloc.argtypes = [pp, i, i, vp, sz, i, i, sp]
        L.flagcxLocalGetDeviceAdaptor.restype = vp
        L.flagcxLocalGetDeviceAdaptor.argtypes = []
        L.flagcxLocalDeviceAdaptorLayout.argtypes = [C.POINTER(sz), i]
        L.flagcxLocalPlanCreate.argtypes = [C.POINTER(vp), i, C.POINTER(i), C.POINTER(i), sz, i, i]
        L.flagcxLocalPlanDestroy.argtypes = [vp]
        L.flagcxLocalPlanImportXml.argtypes = [vp, C.c_char_p]
        L.flagcxLocalPlanExportXml.argtypes = [vp, C.c_char_p]
        L.flagcxLocalPlanSetAlgorithm.argtypes = [vp, i]
        L.flagcxLocalPlanSetFused.argtypes = [vp, i]
        L.flagcxLocalPlanGetTraffic.argtypes = [vp, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        L.flagcxLocalPlanSetChunks.argtypes = [vp, sz]
        szp = C.POINTER(C.c_size_t)
        L.flagcxLocalPlanSetAlltoAllv.argtypes = [vp, szp, szp, szp, szp]
        L.flagcxLocalPlanExecute.argtypes = [vp, pp, pp, pp, i, i, sp]
        L.flagcxLocalPlanGetLastError.restype = C.c_char_p
        L.flagcxLocalPlanGetLastError.argtypes = [vp]
        u64p = C.POINTER(C.c_uint64)
        L.flagcxLocalReduceFifoCreate.argtypes = [C.POINTER(vp), i, i, i, i]
        L.flagcxLocalReduceFifoDestroy.argtypes = [vp]
        L.flagcxLocalReduceFifoStart.argtypes = [vp]
        L.flagcxLocalReduceFifoStop.argtypes = [vp]
        L.flagcxLocalReduceFifoEnqueue.argtypes = [vp, C.POINTER(ReduceTrigger), u64p]
        L.flagcxLocalReduceFifoEnqueueReduce.argtypes = [vp, pp, i, vp, sz, u64p]
        L.flagcxLocalReduceFifoQuery.argtypes = [vp, u64p, u64p, C.POINTER(i)]
        L.flagcxLocalReduceFifoSetOwnQueue.argtypes = [vp, i]
        L.flagcxLocalGateCreate.argtypes = [pp]
        L.flagcxLocalGateDestroy.argtypes = [vp]
        L.flagcxLocalReduceBatchGated.argtypes = [vp, C.POINTER(ReduceDesc), i, i, i, i, sp, u64p]
        L.flagcxLocalGateOpen.argtypes = [vp, C.c_uint64]
        L.flagcxLocalGateQuery.argtypes = [vp, u64p, u64p, C.POINTER(i)]
        L.flagcxLocalGateOwnStream.argtypes = [vp, C.POINTER(sp)]
        L.flagcxLocalReduceFifoWait.argtypes = [vp, C.c_uint64]
        L.flagcxLocalReduceFifoGetGrid.argtypes = [vp, C.POINTER(C.c_uint)]
        L.flagcxLocalReduceFifoSetWaves.argtypes = [vp, i]
        L.flagcxLocalReduceFifoSetLinger.argtypes = [vp, C.c_int64]
        L.flagcxLocalReduceFifoSetWindow.argtypes = [vp, sz]
        L.flagcxLocalReduceFifoGetType.argtypes = [vp, C.POINTER(i), C.POINTER(i), C.POINTER(i)]
        L.flagcxLocalRingReduceScatterFifo.argtypes = [vp, vp, pp, i, i, vp, sz, sp]
        L.flagcxLocalReduceFifoGetLastError.restype = C.c_char_p
        L.flagcxLocalReduceFifoGetLastError.argtypes = [vp]
        L.flagcxLocalSetMaxSpinCount.restype = None
        L.flagcxLocalSetMaxSpinCount.argtypes = [C.c_int64]
        for name in ("deviceAsyncStore", "deviceAsyncLoad"):
            fn = getattr(L, name)
            fn.restype = None
            fn.argtypes = [sp, vp]
        _lib = L
    return _lib


def check(code):
    if code != 0:
        raise FlagcxError(code, lib().flagcxLocalGetLastError().decode())


def type_size(dtype):
    return lib().flagcxLocalGetDataTypeSize(int(dtype))


# ---------------------------------------------------------------- torch side

def _torch():
    import torch
    return torch


def dtype_of(t, bits_as=None):
    """flagcx enum for a torch tensor's dtype (uint16/uint32/uint64 carried as the
    signed tensor type of the same width unless bits_as names the enum)."""
    torch = _torch()
    if bits_as is not None:
        return DataType(bits_as)
    m = {torch.int8: DataType.Int8, torch.uint8: DataType.Uint8, torch.int32: DataType.Int32,
         torch.int64: DataType.Int64, torch.float16: DataType.Float16, torch.float32: DataType.Float32,
         torch.float64: DataType.Float64, torch.bfloat16: DataType.Bfloat16}
    return m[t.dtype]


def current_stream():
    """A flagcxStream wrapper around torch's current HIP stream (not owned)."""
    torch = _torch()
    return Stream(torch.cuda.current_stream().cuda_stream)


def _sref(stream):
    return C.byref(stream) if stream is not None else None


def _ptr_array(ptrs):
    return (C.c_void_p * len(ptrs))(*ptrs)


def place_buffers(pool_ptr, pool_bytes, nbytes, n):
    """Addresses for n buffers of nbytes inside the pool, in different HBM channel groups."""
    out = (C.c_void_p * n)()
    check(lib().flagcxLocalPlaceBuffers(pool_ptr, pool_bytes, nbytes, n, out))
    return [int(p) for p in out]


def reduce(srcs, dst, op, dtype=None, count=None, stream="current"):
    """dst = fold of srcs (torch device tensors) through flagcxLocalReduce."""
    st = current_stream() if stream == "current" else stream
    dt = dtype_of(dst, dtype)
    n = dst.numel() if count is None else count
    check(lib().flagcxLocalReduce(_ptr_array([s.data_ptr() for s in srcs]), len(srcs), dst.data_ptr(), n,
                                  int(dt), int(op), _sref(st)))
    return dst


def reduce_scatter(sendbuffs, rank, recv, op, dtype=None, chunkbytes=None, stream="current"):
    st = current_stream() if stream == "current" else stream
    dt = dtype_of(recv, dtype)
    ptrs = _ptr_array([s.data_ptr() for s in sendbuffs])
    if chunkbytes is None:
        check(lib().flagcxLocalReduceScatter(ptrs, len(sendbuffs), rank, recv.data_ptr(), recv.numel(),
                                             int(dt), int(op), _sref(st)))
    else:
        check(lib().flagcxLocalReduceScatterChunked(ptrs, len(sendbuffs), rank, recv.data_ptr(), recv.numel(),
                                                    int(dt), int(op), chunkbytes, _sref(st)))
    return recv


STATIC_STAGING_BYTES = 8 * 1024 * 1024


def staged_reduce_scatter_noalloc(sendbuffs, rank, recv, op, dtype=None, stream="current"):
    """flagcxLocalStagedReduceScatterNoAlloc: peers' slices staged in the library's static area."""
    st = current_stream() if stream == "current" else stream
    dt = dtype_of(recv, dtype)
    check(lib().flagcxLocalStagedReduceScatterNoAlloc(_ptr_array([s.data_ptr() for s in sendbuffs]), len(sendbuffs),
                                                      rank, recv.data_ptr(), recv.numel(), int(dt), int(op),
                                                      _sref(st)))
    return recv


def all_reduce(sendbuffs, recv, op, dtype=None, stream="current"):
    st = current_stream() if stream == "current" else stream
    dt = dtype_of(recv, dtype)
    check(lib().flagcxLocalAllReduce(_ptr_array([s.data_ptr() for s in sendbuffs]), len(sendbuffs),
                                     recv.data_ptr(), recv.numel(), int(dt), int(op), _sref(st)))
    return recv


def reduce_batch(descs, op, dtype, nranks, stream="current"):
    """descs: list of (list_of_src_ptrs, dst_ptr, count).  One flagcxLocalReduceBatch call."""
    st = current_stream() if stream == "current" else stream
    keep = [_ptr_array(list(d[0])) for d in descs]
    arr = (ReduceDesc * len(descs))(*[ReduceDesc(keep[i], d[1], d[2]) for i, d in enumerate(descs)])
    check(lib().flagcxLocalReduceBatch(arr, len(descs), nranks, int(dtype), int(op), _sref(st)))


def reduce_batch_sparse(descs, op, dtype, nlive, nzero, stream="current"):
    """descs as reduce_batch, each listing the nlive members that hold data; nzero more members hold zeros."""
    st = current_stream() if stream == "current" else stream
    keep = [_ptr_array(list(d[0])) for d in descs]
    arr = (ReduceDesc * len(descs))(*[ReduceDesc(keep[i], d[1], d[2]) for i, d in enumerate(descs)])
    check(lib().flagcxLocalReduceBatchSparse(arr, len(descs), nlive, nzero, int(dtype), int(op), _sref(st)))


def reduce_triggers(triggers, stream="current"):
    st = current_stream() if stream == "current" else stream
    arr = (ReduceTrigger * len(triggers))(*triggers)
    check(lib().flagcxLocalReduceTriggers(arr, len(triggers), _sref(st)))


def ring_chunk_table(count, dtype, nranks):
    off = (C.c_size_t * nranks)()
    ln = (C.c_size_t * nranks)()
    check(lib().flagcxLocalRingChunkTable(count, int(dtype), nranks, off, ln))
    return list(off), list(ln)


def memcpy(dst_ptr, src_ptr, size, stream="current"):
    st = current_stream() if stream == "current" else stream
    check(lib().flagcxLocalMemcpy(dst_ptr, src_ptr, size, _sref(st)))


def memset(ptr, value, size, stream="current"):
    st = current_stream() if stream == "current" else stream
    check(lib().flagcxLocalMemset(ptr, value, size, _sref(st)))


def refresh(buff, start, offset, count, totalcount, op, dtype=None, stream="current"):
    st = current_stream() if stream == "current" else stream
    dt = dtype_of(buff, dtype)
    check(lib().flagcxLocalRefresh(buff.data_ptr(), start, offset, count, totalcount, int(dt), int(op), _sref(st)))


def pack(dst_ptr, src_ptr, nchunks, chunkbytes, srcstride, stream="current"):
    st = current_stream() if stream == "current" else stream
    check(lib().flagcxLocalPack(dst_ptr, src_ptr, nchunks, chunkbytes, srcstride, _sref(st)))


def unpack(dst_ptr, src_ptr, nchunks, chunkbytes, dststride, stream="current"):
    st = current_stream() if stream == "current" else stream
    check(lib().flagcxLocalUnpack(dst_ptr, src_ptr, nchunks, chunkbytes, dststride, _sref(st)))


def pack_list(dst_ptr, src_ptrs, nbytes, stream="current"):
    st = current_stream() if stream == "current" else stream
    check(lib().flagcxLocalPackList(dst_ptr, _ptr_array(src_ptrs), len(src_ptrs), nbytes, _sref(st)))


def unpack_list(dst_ptrs, src_ptr, nbytes, stream="current"):
    st = current_stream() if stream == "current" else stream
    check(lib().flagcxLocalUnpackList(_ptr_array(dst_ptrs), src_ptr, len(dst_ptrs), nbytes, _sref(st)))


def copy_fanout(copies, stream="current"):
    """copies: list of (src_ptr, list_of_dst_ptrs, nbytes).  One flagcxLocalCopyFanout call."""
    st = current_stream() if stream == "current" else stream
    keep = [_ptr_array(list(c[1])) for c in copies]
    arr = (FanoutDesc * len(copies))(*[FanoutDesc(c[0], keep[i], len(c[1]), c[2]) for i, c in enumerate(copies)])
    check(lib().flagcxLocalCopyFanout(arr, len(copies), _sref(st)))


class Plan:
    """A set of per-rank C2C plans replayed on one GPU (flagcxLocalPlan*)."""

    def __init__(self, cluster_ids, total_count, comm_op, red_op, is_inter=None):
        n = len(cluster_ids)
        self.nranks = n
        self._h = C.c_void_p()
        cl = (C.c_int * n)(*cluster_ids)
        it = (C.c_int * n)(*is_inter) if is_inter is not None else None
        rc = lib().flagcxLocalPlanCreate(C.byref(self._h), n, cl, it, total_count, int(comm_op), int(red_op))
        if rc:
            raise FlagcxError(rc, "flagcxLocalPlanCreate")

    def _check(self, rc):
        if rc:
            raise FlagcxError(rc, lib().flagcxLocalPlanGetLastError(self._h).decode() or
                              lib().flagcxLocalGetLastError().decode())

    def import_xml(self, prefix):
        self._check(lib().flagcxLocalPlanImportXml(self._h, prefix.encode()))

    def export_xml(self, prefix):
        self._check(lib().flagcxLocalPlanExportXml(self._h, prefix.encode()))

    def set_chunks(self, nchunks):
        self._check(lib().flagcxLocalPlanSetChunks(self._h, nchunks))

    def set_alltoallv(self, send_counts, s_displs, recv_counts, r_displs):
        """Four nranks x nranks matrices (nested lists), row r = rank r's arrays, in elements."""
        def flat(m):
            if m is None:
                return None
            v = [int(x) for row in m for x in row]
            return (C.c_size_t * len(v))(*v)
        self._check(lib().flagcxLocalPlanSetAlltoAllv(self._h, flat(send_counts), flat(s_displs), flat(recv_counts),
                                                      flat(r_displs)))

    def set_algorithm(self, algo):
        self._check(lib().flagcxLocalPlanSetAlgorithm(self._h, algo))

    def set_fused(self, fused):
        """True (default): refreshes are recorded and sums skip the cleared members; False: literal replay."""
        self._check(lib().flagcxLocalPlanSetFused(self._h, 1 if fused else 0))

    def traffic(self):
        """(algorithmic bytes, kernel launches) of the last execute."""
        b, n = C.c_uint64(), C.c_uint64()
        self._check(lib().flagcxLocalPlanGetTraffic(self._h, C.byref(b), C.byref(n)))
        return b.value, n.value

    def execute(self, send_ptrs, recv_ptrs, scratch_ptrs, dtype, root=-1, stream="current"):
        st = current_stream() if stream == "current" else stream
        sc = _ptr_array(scratch_ptrs) if scratch_ptrs is not None else None
        self._check(lib().flagcxLocalPlanExecute(self._h, _ptr_array(send_ptrs), _ptr_array(recv_ptrs), sc,
                                                 int(dtype), root, _sref(st)))

    def close(self):
        if self._h:
            lib().flagcxLocalPlanDestroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Ring:
    """Staging ring over caller memory (flagcxLocalRing*); ring_tensor stays referenced."""

    def __init__(self, ring_tensor, npeers, chunkbytes=0, steps=0):
        self._keep = ring_tensor
        self._h = C.c_void_p()
        rc = lib().flagcxLocalRingCreate(C.byref(self._h), ring_tensor.data_ptr(),
                                         ring_tensor.numel() * ring_tensor.element_size(), npeers, chunkbytes, steps)
        if rc:
            raise FlagcxError(rc, "flagcxLocalRingCreate")

    def send_recv(self, dst_ptr, src_ptr, size, copy_stream, stream):
        check(lib().flagcxLocalRingSendRecv(self._h, dst_ptr, src_ptr, size, C.byref(copy_stream), C.byref(stream)))

    def reduce_scatter(self, sendbuffs, rank, recv, op, copy_stream, stream, dtype=None):
        dt = dtype_of(recv, dtype)
        check(lib().flagcxLocalRingReduceScatter(self._h, _ptr_array([s.data_ptr() for s in sendbuffs]),
                                                 len(sendbuffs), rank, recv.data_ptr(), recv.numel(), int(dt),
                                                 int(op), C.byref(copy_stream), C.byref(stream)))

    def reduce_scatter_fifo(self, fifo, sendbuffs, rank, recv, copy_stream):
        """Proxy-style: staging copies on copy_stream, reduces through the running ReduceFifo; blocks."""
        rc = lib().flagcxLocalRingReduceScatterFifo(self._h, fifo._h, _ptr_array([s.data_ptr() for s in sendbuffs]),
                                                    len(sendbuffs), rank, recv.data_ptr(), recv.numel(),
                                                    C.byref(copy_stream))
        if rc:
            raise FlagcxError(rc, (lib().flagcxLocalReduceFifoGetLastError(fifo._h) or b"").decode())

    def close(self):
        if self._h:
            lib().flagcxLocalRingDestroy(self._h)
            self._h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Gate:
    """A count that the host raises as the inputs of a gated batch complete (flagcxLocalGate*)."""

    def __init__(self):
        self._h = C.c_void_p()
        check(lib().flagcxLocalGateCreate(C.byref(self._h)))

    def reduce_batch(self, descs, op, dtype, nranks, stream="current"):
        """descs as reduce_batch; launched now, folded as open() passes each descriptor's number.
        Returns the number of descs[0]."""
        st = current_stream() if stream == "current" else stream
        keep = [_ptr_array(list(d[0])) for d in descs]
        arr = (ReduceDesc * len(descs))(*[ReduceDesc(keep[i], d[1], d[2]) for i, d in enumerate(descs)])
        first = C.c_uint64()
        check(lib().flagcxLocalReduceBatchGated(self._h, arr, len(descs), nranks, int(dtype), int(op), _sref(st),
                                                C.byref(first)))
        return first.value

    def open(self, upto):
        check(lib().flagcxLocalGateOpen(self._h, upto))

    def own_stream(self):
        """The gate's stream (a Stream structure): a hardware queue that nothing else shares."""
        p = C.POINTER(Stream)()
        check(lib().flagcxLocalGateOwnStream(self._h, C.byref(p)))
        return p.contents

    def query(self):
        """(descriptors numbered so far, count, state)."""
        a, b, st = C.c_uint64(), C.c_uint64(), C.c_int()
        check(lib().flagcxLocalGateQuery(self._h, C.byref(a), C.byref(b), C.byref(st)))
        return a.value, b.value, st.value

    def destroy(self):
        if self._h:
            h, self._h = self._h, C.c_void_p()
            check(lib().flagcxLocalGateDestroy(h))

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.destroy()
        return False


class ReduceFifo:
    """Host-producer / device-consumer reduce queue (flagcxLocalReduceFifo*).

    The consumer kernel is on the GPU while entries are outstanding and for a short linger
    after; then it parks and the next entry launches it again.  Use the object as a context
    manager so that an exception between start and stop still stops it.
    """

    def __init__(self, capacity, max_ranks, dtype, op):
        self._h = C.c_void_p()
        rc = lib().flagcxLocalReduceFifoCreate(C.byref(self._h), capacity, max_ranks, int(dtype), int(op))
        if rc:
            raise FlagcxError(rc, "flagcxLocalReduceFifoCreate")

    def _check(self, rc):
        if rc:
            raise FlagcxError(rc, (lib().flagcxLocalReduceFifoGetLastError(self._h) or b"").decode())

    def start(self):
        self._check(lib().flagcxLocalReduceFifoStart(self._h))
        return self

    def stop(self):
        self._check(lib().flagcxLocalReduceFifoStop(self._h))

    def try_enqueue_reduce(self, src_ptrs, dst_ptr, count):
        """Ticket, or None when the ring is full."""
        t = C.c_uint64()
        rc = lib().flagcxLocalReduceFifoEnqueueReduce(self._h, _ptr_array(src_ptrs), len(src_ptrs), dst_ptr, count,
                                                      C.byref(t))
        if rc == Result.InProgress:
            return None
        self._check(rc)
        return t.value

    def enqueue_reduce(self, src_ptrs, dst_ptr, count):
        while True:
            t = self.try_enqueue_reduce(src_ptrs, dst_ptr, count)
            if t is not None:
                return t

    def enqueue(self, trigger):
        t = C.c_uint64()
        while True:
            rc = lib().flagcxLocalReduceFifoEnqueue(self._h, C.byref(trigger), C.byref(t))
            if rc != Result.InProgress:
                break
        self._check(rc)
        return t.value

    def query(self):
        """(produced, consumed, state)"""
        p, c, st = C.c_uint64(), C.c_uint64(), C.c_int()
        self._check(lib().flagcxLocalReduceFifoQuery(self._h, C.byref(p), C.byref(c), C.byref(st)))
        return p.value, c.value, st.value

    def wait(self, ticket):
        self._check(lib().flagcxLocalReduceFifoWait(self._h, ticket))

    def set_window(self, nbytes):
        self._check(lib().flagcxLocalReduceFifoSetWindow(self._h, nbytes))

    def set_own_queue(self, own=True):
        """A hardware queue of its own for the consumer (its stream then is a blocking one)."""
        self._check(lib().flagcxLocalReduceFifoSetOwnQueue(self._h, 1 if own else 0))

    def set_linger(self, polls):
        self._check(lib().flagcxLocalReduceFifoSetLinger(self._h, polls))

    def set_waves(self, waves_per_cu):
        self._check(lib().flagcxLocalReduceFifoSetWaves(self._h, waves_per_cu))

    def grid(self):
        g = C.c_uint()
        self._check(lib().flagcxLocalReduceFifoGetGrid(self._h, C.byref(g)))
        return g.value

    def close(self):
        if self._h:
            lib().flagcxLocalReduceFifoDestroy(self._h)
            self._h = C.c_void_p()

    def __enter__(self):
        return self.start()

    def __exit__(self, *exc):
        try:
            lib().flagcxLocalReduceFifoStop(self._h)
        finally:
            return False

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


ADAPTOR_SLOTS = [
    "deviceSynchronize", "deviceMemcpy", "deviceMemset", "deviceMalloc", "deviceFree", "setDevice", "getDevice",
    "getDeviceCount", "getVendor", "hostGetDevicePointer", "memHandleInit", "memHandleDestroy", "gdrMemAlloc",
    "gdrMemFree", "hostShareMemAlloc", "hostShareMemFree", "gdrPtrMmap", "gdrPtrMunmap", "streamCreate",
    "streamDestroy", "streamCopy", "streamFree", "streamSynchronize", "streamQuery", "streamWaitEvent",
    "eventCreate", "eventDestroy", "eventRecord", "eventSynchronize", "eventQuery", "ipcMemHandleCreate",
    "ipcMemHandleGet", "ipcMemHandleOpen", "ipcMemHandleClose", "ipcMemHandleFree", "launchKernel", "copyArgsInit",
    "copyArgsFree", "launchDeviceFunc", "getDeviceProperties", "getDevicePciBusId", "getDeviceByPciBusId",
    "launchHostFunc", "dmaSupport", "getHandleForAddressRange", "eventElapsedTime",
]


def device_adaptor():
    """(name, {slot: address or None}) of the exported flagcxDeviceAdaptor table."""
    base = lib().flagcxLocalGetDeviceAdaptor()
    name = C.string_at(base, 32).split(b"\0")[0].decode()
    ptrs = (C.c_void_p * len(ADAPTOR_SLOTS)).from_address(base + 32)
    return name, {n: ptrs[k] for k, n in enumerate(ADAPTOR_SLOTS)}


def adaptor_fn(slots, name, restype, *argtypes):
    return C.CFUNCTYPE(restype, *argtypes)(slots[name])
