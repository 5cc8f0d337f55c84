"""The HIP device-adaptor table exercised slot by slot through its function
pointers, the way the reference's core calls deviceAdaptor->...()."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

H2D, D2H, D2D = 0, 1, 2
MEM_HOST, MEM_DEVICE, MEM_MANAGED = 0, 1, 2
IN_PROGRESS = 7


@pytest.fixture(scope="module")
def A():
    import torch
    assert torch.cuda.is_available()
    torch.cuda.init()
    from flagcx_amd import local
    name, slots = local.device_adaptor()
    vp, i, sz = C.c_void_p, C.c_int, C.c_size_t
    f = lambda n, *a: local.adaptor_fn(slots, n, i, *a)

    class T:
        pass
    t = T()
    t.local = local
    t.sync = f("deviceSynchronize")
    t.memcpy = f("deviceMemcpy", vp, vp, sz, i, vp, vp)
    t.memset = f("deviceMemset", vp, i, sz, i, vp)
    t.malloc = f("deviceMalloc", C.POINTER(vp), sz, i, vp)
    t.free = f("deviceFree", vp, i, vp)
    t.set_device = f("setDevice", i)
    t.get_device = f("getDevice", C.POINTER(i))
    t.get_count = f("getDeviceCount", C.POINTER(i))
    t.host_ptr = f("hostGetDevicePointer", C.POINTER(vp), vp)
    t.gdr_alloc = f("gdrMemAlloc", C.POINTER(vp), sz, vp)
    t.gdr_free = f("gdrMemFree", vp, vp)
    t.s_create = f("streamCreate", C.POINTER(vp))
    t.s_destroy = f("streamDestroy", vp)
    t.s_copy = f("streamCopy", C.POINTER(vp), vp)
    t.s_free = f("streamFree", vp)
    t.s_sync = f("streamSynchronize", vp)
    t.s_query = f("streamQuery", vp)
    t.s_wait = f("streamWaitEvent", vp, vp)
    t.e_create = f("eventCreate", C.POINTER(vp), i)
    t.e_destroy = f("eventDestroy", vp)
    t.e_record = f("eventRecord", vp, vp)
    t.e_sync = f("eventSynchronize", vp)
    t.e_query = f("eventQuery", vp)
    t.e_elapsed = f("eventElapsedTime", C.POINTER(C.c_float), vp, vp)
    t.ipc_create = f("ipcMemHandleCreate", C.POINTER(vp), C.POINTER(sz))
    t.ipc_get = f("ipcMemHandleGet", vp, vp)
    t.ipc_free = f("ipcMemHandleFree", vp)
    t.launch_dev = f("launchDeviceFunc", vp, vp, vp)
    t.launch_host = f("launchHostFunc", vp, vp, vp)
    t.props = f("getDeviceProperties", vp, i)
    t.pci_of = f("getDevicePciBusId", C.c_char_p, i, i)
    t.by_pci = f("getDeviceByPciBusId", C.POINTER(i), C.c_char_p)
    t.dmabuf = f("getHandleForAddressRange", vp, vp, sz, C.c_ulonglong)
    return t


def test_memory_copy_set_paths(A):
    n = 1 << 20
    dev = C.c_void_p()
    dev2 = C.c_void_p()
    host = C.c_void_p()
    st = C.c_void_p()
    assert A.s_create(C.byref(st)) == 0
    assert A.malloc(C.byref(dev), n, MEM_DEVICE, None) == 0
    assert A.malloc(C.byref(dev2), n, MEM_DEVICE, st) == 0          # stream-ordered allocation
    assert A.malloc(C.byref(host), n, MEM_HOST, None) == 0
    src = np.random.default_rng(0).integers(0, 256, n, dtype=np.uint8)
    C.memmove(host, src.ctypes.data, n)
    assert A.memcpy(dev, host, n, H2D, st, None) == 0
    assert A.memcpy(dev2, dev, n, D2D, st, None) == 0                # this library's copy kernel
    assert A.memset(dev, 0x5A, n // 2, MEM_DEVICE, st) == 0         # this library's fill kernel
    assert A.memset(host, 0, n, MEM_HOST, None) == 0
    assert A.s_sync(st) == 0 and A.s_query(st) == 0
    out = np.empty(n, dtype=np.uint8)
    assert A.memcpy(out.ctypes.data, dev2, n, D2H, None, None) == 0  # NULL stream: blocking
    assert out.tobytes() == src.tobytes()
    assert A.memcpy(out.ctypes.data, dev, n, D2H, None, None) == 0
    assert (out[:n // 2] == 0x5A).all() and out[n // 2:].tobytes() == src[n // 2:].tobytes()
    assert A.memcpy(dev, host, n, 9, st, None) == 4
    dp = C.c_void_p()
    assert A.host_ptr(C.byref(dp), host) == 0 and dp.value
    g = C.c_void_p()
    assert A.gdr_alloc(C.byref(g), 4096, None) == 0 and A.gdr_free(g, None) == 0
    m = C.c_void_p()
    assert A.malloc(C.byref(m), 4096, MEM_MANAGED, None) == 0 and A.free(m, MEM_MANAGED, None) == 0
    assert A.free(dev2, MEM_DEVICE, st) == 0
    assert A.s_sync(st) == 0
    assert A.free(dev, MEM_DEVICE, None) == 0 and A.free(host, MEM_HOST, None) == 0
    assert A.free(None, MEM_DEVICE, None) == 0
    assert A.s_destroy(st) == 0
    assert A.sync() == 0


def test_streams_events_and_funcs(A):
    import torch
    st = C.c_void_p()
    assert A.s_create(C.byref(st)) == 0
    e0, e1 = C.c_void_p(), C.c_void_p()
    assert A.e_create(C.byref(e0), 0) == 0 and A.e_create(C.byref(e1), 0) == 0
    buf = torch.zeros(1 << 22, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    assert A.e_record(e0, st) == 0
    assert A.memset(buf.data_ptr(), 7, buf.numel(), MEM_DEVICE, st) == 0
    assert A.e_record(e1, st) == 0
    assert A.e_sync(e1) == 0 and A.e_query(e1) == 0
    ms = C.c_float(-1)
    assert A.e_elapsed(C.byref(ms), e0, e1) == 0 and ms.value > 0
    assert int(buf.sum().item()) == 7 * buf.numel()
    # a wrapper around a foreign stream: not owned, only the wrapper is freed
    ts = torch.cuda.Stream()
    raw = C.c_void_p(ts.cuda_stream)
    wrapped = C.c_void_p()
    assert A.s_copy(C.byref(wrapped), C.byref(raw)) == 0
    assert A.s_wait(wrapped, e1) == 0
    flag = torch.zeros(1, dtype=torch.uint8, device="cuda")
    store = C.cast(A.local.lib().deviceAsyncStore, C.c_void_p)
    assert A.launch_dev(wrapped, store, flag.data_ptr()) == 0
    assert A.s_sync(wrapped) == 0 and flag.item() == 1
    hits = []
    cb = C.CFUNCTYPE(None, C.c_void_p)(lambda a: hits.append(a))
    assert A.launch_host(wrapped, cb, 42) == 0
    assert A.s_sync(wrapped) == 0 and hits == [42]
    assert A.s_free(wrapped) == 0
    ts.synchronize()                                     # the foreign stream is still alive
    notime = C.c_void_p()
    assert A.e_create(C.byref(notime), 1) == 0 and A.e_record(notime, None) == 0 and A.e_sync(notime) == 0
    for e in (e0, e1, notime):
        assert A.e_destroy(e) == 0
    assert A.s_destroy(st) == 0


def test_device_queries_and_ipc_handle(A):
    import torch
    d, n = C.c_int(-1), C.c_int(-1)
    assert A.get_device(C.byref(d)) == 0 and A.get_count(C.byref(n)) == 0 and 0 <= d.value < n.value
    assert A.set_device(d.value) == 0
    props = C.create_string_buffer(256 + 12)
    assert A.props(props, d.value) == 0 and len(props.raw[:256].split(b"\0")[0]) > 0
    bus = C.create_string_buffer(64)
    assert A.pci_of(bus, 64, d.value) == 0 and b":" in bus.value
    back = C.c_int(-1)
    assert A.by_pci(C.byref(back), bus.value) == 0 and back.value == d.value
    h, sz = C.c_void_p(), C.c_size_t(0)
    assert A.ipc_create(C.byref(h), C.byref(sz)) == 0 and sz.value == 64
    mem = C.c_void_p()
    hip_malloc = A.malloc
    assert hip_malloc(C.byref(mem), 1 << 20, MEM_DEVICE, None) == 0
    assert A.ipc_get(h, mem) == 0
    assert A.ipc_get(h, None) == 4
    assert A.ipc_free(h) == 0
    assert A.free(mem, MEM_DEVICE, None) == 0
    assert A.dmabuf(None, None, 0, 0) == 9


def test_cpp_collective_test_program():
    """The C++ caller test (reference unit-test patterns over 8 simulated ranks,
    buffers from the device-adaptor table) passes."""
    import os
    import subprocess
    from flagcx_amd import local
    exe = os.path.join(os.path.dirname(local.lib_path()), "local_coll_test")
    assert os.path.exists(exe), "build it with python -m flagcx_amd.build"
    r = subprocess.run([exe, "-n", "8", "-c", str(1 << 22)], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "PASSED" in r.stdout and r.stdout.count("ok ") == 7
