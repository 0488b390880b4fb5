"""Device-adaptor plugin conformance on a real GPU, case for case after the
reference's single-GPU adaptor test (test/unittest/adaptor/test_device_adaptor.cpp:49-730),
driven through the plugin's function table as FlagCX's loader would hand it out."""
import ctypes as C
import re
import time

import numpy as np
import pytest

from flagcx_amd import _native as N
from flagcx_amd.adaptor import HOST_FUNC, LAUNCH_FUNC, DevProps

pytestmark = pytest.mark.gpu

TEST_COUNT = 1024
TEST_SIZE = TEST_COUNT * 4
OK = N.SUCCESS


@pytest.fixture()
def t(dev):
    return dev.t


@pytest.fixture()
def stream(dev):
    s = dev.stream_create()
    yield s
    dev.stream_destroy(s)


def _malloc(t, size, kind, stream=None):
    p = C.c_void_p()
    assert t.deviceMalloc(C.byref(p), size, kind, stream) == OK and p.value
    return p.value


def _host_view(ptr, count, ctype=C.c_float):
    return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(ctype)), shape=(count,))


def test_get_device_info(t):                                    # :49-68
    n, d = C.c_int(), C.c_int(-1)
    assert t.getDeviceCount(C.byref(n)) == OK and n.value > 0
    assert t.getDevice(C.byref(d)) == OK and d.value == 0
    v = C.create_string_buffer(128)
    assert t.getVendor(v) == OK and v.value == b"AMD"


def test_device_and_host_alloc(t, stream):                      # :70-98
    p = _malloc(t, TEST_SIZE, N.MEM_DEVICE, stream)             # stream-ordered allocation
    assert t.deviceFree(p, N.MEM_DEVICE, stream) == OK
    h = _malloc(t, TEST_SIZE, N.MEM_HOST, stream)
    assert t.deviceFree(h, N.MEM_HOST, stream) == OK
    m = _malloc(t, TEST_SIZE, N.MEM_MANAGED)
    assert t.deviceFree(m, N.MEM_MANAGED, None) == OK
    assert t.streamSynchronize(stream) == OK


def test_memory_copy_round_trip(t, stream):                     # :100-149
    src, dst = _malloc(t, TEST_SIZE, N.MEM_HOST), _malloc(t, TEST_SIZE, N.MEM_HOST)
    d = _malloc(t, TEST_SIZE, N.MEM_DEVICE)
    _host_view(src, TEST_COUNT)[:] = np.arange(TEST_COUNT, dtype=np.float32)
    _host_view(dst, TEST_COUNT)[:] = 0
    assert t.deviceMemcpy(d, src, TEST_SIZE, N.MEMCPY_H2D, stream, None) == OK
    assert t.deviceMemcpy(dst, d, TEST_SIZE, N.MEMCPY_D2H, stream, None) == OK
    assert t.streamSynchronize(stream) == OK
    assert np.array_equal(_host_view(dst, TEST_COUNT), np.arange(TEST_COUNT, dtype=np.float32))
    for p, k in ((src, N.MEM_HOST), (dst, N.MEM_HOST), (d, N.MEM_DEVICE)):
        assert t.deviceFree(p, k, None) == OK


def test_memory_set(t, stream):                                 # :151-185
    d, h = _malloc(t, TEST_SIZE, N.MEM_DEVICE), _malloc(t, TEST_SIZE, N.MEM_HOST)
    assert t.deviceMemset(d, 0, TEST_SIZE, N.MEM_DEVICE, stream) == OK
    assert t.deviceMemcpy(h, d, TEST_SIZE, N.MEMCPY_D2H, stream, None) == OK
    assert t.streamSynchronize(stream) == OK
    assert (_host_view(h, TEST_SIZE, C.c_ubyte) == 0).all()
    assert t.deviceMemset(d, 0xAB, TEST_SIZE, N.MEM_DEVICE, None) == OK           # synchronous form
    assert t.deviceMemcpy(h, d, TEST_SIZE, N.MEMCPY_D2H, None, None) == OK
    assert (_host_view(h, TEST_SIZE, C.c_ubyte) == 0xAB).all()
    assert t.deviceMemset(h, 0x11, TEST_SIZE, N.MEM_HOST, None) == OK             # host memory: plain memset
    assert (_host_view(h, TEST_SIZE, C.c_ubyte) == 0x11).all()
    assert t.deviceFree(d, N.MEM_DEVICE, None) == OK and t.deviceFree(h, N.MEM_HOST, None) == OK


def test_stream_operations(t):                                  # :187-208
    s = C.c_void_p()
    assert t.streamCreate(C.byref(s)) == OK and s.value
    assert t.streamSynchronize(s) == OK
    assert t.streamQuery(s) == OK                               # idle stream: done, not in progress
    assert t.streamDestroy(s) == OK


def test_event_operations(t, stream):                           # :210-234
    for kind in (0, 1):                                         # default, disable-timing
        e = C.c_void_p()
        assert t.eventCreate(C.byref(e), kind) == OK and e.value
        assert t.eventRecord(e, stream) == OK
        assert t.eventSynchronize(e) == OK
        assert t.eventQuery(e) == OK
        assert t.eventDestroy(e) == OK


def test_stream_wait_event(t, stream):                          # :236-262
    s2, e = C.c_void_p(), C.c_void_p()
    assert t.streamCreate(C.byref(s2)) == OK and t.eventCreate(C.byref(e), 1) == OK
    assert t.eventRecord(e, stream) == OK
    assert t.streamWaitEvent(s2, e) == OK
    assert t.streamSynchronize(s2) == OK and t.streamSynchronize(stream) == OK
    assert t.eventDestroy(e) == OK and t.streamDestroy(s2) == OK


def test_device_synchronize_and_set_device(t):                  # :264-294
    assert t.deviceSynchronize() == OK
    n, d = C.c_int(), C.c_int(-1)
    t.getDeviceCount(C.byref(n))
    for i in range(n.value):
        assert t.setDevice(i) == OK
        assert t.getDevice(C.byref(d)) == OK and d.value == i
    assert t.setDevice(0) == OK
    assert t.setDevice(n.value) != OK                           # out of range is an error, not a crash
    assert t.setDevice(0) == OK


def test_large_alloc(t):                                        # :296-319 (256 MiB there; 1 GiB here)
    p = _malloc(t, 1 << 30, N.MEM_DEVICE)
    assert t.deviceMemset(p, 0, 1 << 30, N.MEM_DEVICE, None) == OK
    assert t.deviceFree(p, N.MEM_DEVICE, None) == OK


def test_event_timing(t, stream):                               # :321-360, :624-649
    e0, e1 = C.c_void_p(), C.c_void_p()
    assert t.eventCreate(C.byref(e0), 0) == OK and t.eventCreate(C.byref(e1), 0) == OK
    d = _malloc(t, 64 << 20, N.MEM_DEVICE)
    assert t.eventRecord(e0, stream) == OK
    for _ in range(4):
        assert t.deviceMemset(d, 1, 64 << 20, N.MEM_DEVICE, stream) == OK
    assert t.eventRecord(e1, stream) == OK
    assert t.eventSynchronize(e1) == OK
    ms = C.c_float(-1)
    assert t.eventElapsedTime(C.byref(ms), e0, e1) == OK and 0 < ms.value < 1000
    assert t.eventElapsedTime(None, e0, e1) == N.INVALID_ARGUMENT
    assert t.eventElapsedTime(C.byref(ms), None, e1) == N.INVALID_ARGUMENT
    assert t.eventElapsedTime(C.byref(ms), e0, None) == N.INVALID_ARGUMENT
    assert t.eventDestroy(e0) == OK and t.eventDestroy(e1) == OK
    assert t.deviceFree(d, N.MEM_DEVICE, None) == OK


def test_device_to_device_memcpy(t, stream):                    # :362-414
    h = _malloc(t, TEST_SIZE, N.MEM_HOST)
    a, b = _malloc(t, TEST_SIZE, N.MEM_DEVICE), _malloc(t, TEST_SIZE, N.MEM_DEVICE)
    _host_view(h, TEST_COUNT)[:] = np.arange(TEST_COUNT, dtype=np.float32) * 2
    assert t.deviceMemcpy(a, h, TEST_SIZE, N.MEMCPY_H2D, stream, None) == OK
    assert t.deviceMemcpy(b, a, TEST_SIZE, N.MEMCPY_D2D, stream, None) == OK
    assert t.streamSynchronize(stream) == OK                    # pinned source is read asynchronously
    _host_view(h, TEST_COUNT)[:] = 0
    assert t.deviceMemcpy(h, b, TEST_SIZE, N.MEMCPY_D2H, None, None) == OK
    assert np.array_equal(_host_view(h, TEST_COUNT), np.arange(TEST_COUNT, dtype=np.float32) * 2)
    for p, k in ((h, N.MEM_HOST), (a, N.MEM_DEVICE), (b, N.MEM_DEVICE)):
        assert t.deviceFree(p, k, None) == OK


def test_stream_copy_and_free(t, stream, dev):                  # :416-444
    raw = dev.raw_stream(stream)
    wrapped = C.c_void_p()
    assert t.streamCopy(C.byref(wrapped), raw) == OK and wrapped.value
    assert dev.raw_stream(wrapped.value) == raw                 # same underlying stream, not owned
    assert t.streamSynchronize(wrapped) == OK
    assert t.streamFree(wrapped) == OK                          # frees the wrapper only
    assert t.streamSynchronize(stream) == OK                    # original still usable


def test_host_get_device_pointer(t):                            # :446-466
    h = _malloc(t, TEST_SIZE, N.MEM_HOST)
    d = C.c_void_p()
    assert t.hostGetDevicePointer(C.byref(d), h) == OK and d.value
    assert t.hostGetDevicePointer(None, h) == N.INVALID_ARGUMENT
    assert t.hostGetDevicePointer(C.byref(d), None) == N.INVALID_ARGUMENT
    # the device pointer really aliases the pinned buffer: a device memset shows up on the host
    assert t.deviceMemset(d, 0x5C, TEST_SIZE, N.MEM_DEVICE, None) == OK
    assert t.deviceSynchronize() == OK
    assert (_host_view(h, TEST_SIZE, C.c_ubyte) == 0x5C).all()
    assert t.deviceFree(h, N.MEM_HOST, None) == OK


def test_pci_bus_id_and_properties(t):                          # :512-622
    n = C.c_int()
    t.getDeviceCount(C.byref(n))
    for i in range(n.value):
        buf = C.create_string_buffer(64)
        assert t.getDevicePciBusId(buf, 64, i) == OK
        assert re.fullmatch(rb"[0-9a-fA-F]+:[0-9a-fA-F]+:[0-9a-fA-F]+\.[0-9a-fA-F]+", buf.value), buf.value
        back = C.c_int(-1)
        assert t.getDeviceByPciBusId(C.byref(back), buf.value) == OK and back.value == i
        props = DevProps()
        assert t.getDeviceProperties(C.byref(props), i) == OK and props.name
        dom, bus, devid = (int(x, 16) for x in re.split(rb"[:.]", buf.value)[:3])
        assert (props.pciDomainId, props.pciBusId, props.pciDeviceId) == (dom, bus, devid)
    buf = C.create_string_buffer(64)
    assert t.getDevicePciBusId(None, 64, 0) == N.INVALID_ARGUMENT
    assert t.getDevicePciBusId(buf, 64, -1) != OK and t.getDevicePciBusId(buf, 64, n.value) != OK
    assert t.getDeviceProperties(None, 0) == N.INVALID_ARGUMENT
    assert t.getDeviceProperties(C.byref(DevProps()), n.value) != OK
    assert t.getDeviceByPciBusId(None, b"0000:00:00.0") == N.INVALID_ARGUMENT
    assert t.deviceSynchronize() == OK                          # no sticky error left behind


def test_ipc_mem_handles(t):                                    # :651-728
    h, size = C.c_void_p(), C.c_size_t()
    assert t.ipcMemHandleCreate(C.byref(h), C.byref(size)) == OK and h.value and size.value > 0
    d = _malloc(t, 4096, N.MEM_DEVICE)
    assert t.ipcMemHandleGet(h, d) == OK                        # the reference's HIP adaptor returns NotSupported here
    assert t.ipcMemHandleGet(None, d) == N.INVALID_ARGUMENT
    assert t.ipcMemHandleGet(h, None) == N.INVALID_ARGUMENT
    assert t.ipcMemHandleClose(None) == N.INVALID_ARGUMENT
    already = C.c_void_p(1)
    assert t.ipcMemHandleOpen(h, C.byref(already)) == N.INVALID_ARGUMENT         # *devPtr must be NULL
    assert t.ipcMemHandleFree(h) == OK
    h2 = C.c_void_p()
    assert t.ipcMemHandleCreate(C.byref(h2), None) == OK and t.ipcMemHandleFree(h2) == OK
    assert t.deviceFree(d, N.MEM_DEVICE, None) == OK


def test_launch_device_func_and_host_func(t, stream, dev):      # hot-path hooks: group.cc:451-453
    seen = []

    @LAUNCH_FUNC
    def enqueue(s, args):                                       # a "device function": enqueues work on the stream it gets
        seen.append((s, args))
        t.deviceMemset(args, 0x42, 256, N.MEM_DEVICE, s)

    d = _malloc(t, 256, N.MEM_DEVICE)
    assert t.launchDeviceFunc(stream, enqueue, d) == OK
    assert seen == [(stream, d)]
    fired = []

    @HOST_FUNC
    def cb(arg):
        fired.append(arg)

    assert t.launchHostFunc(stream, cb, 7) == OK
    assert t.streamSynchronize(stream) == OK
    deadline = time.time() + 5
    while not fired and time.time() < deadline:
        time.sleep(0.01)
    assert fired == [7]
    assert (dev.to_host(d, 256, np.uint8) == 0x42).all()
    assert t.deviceFree(d, N.MEM_DEVICE, None) == OK


def test_stream_write_and_wait_value(t, stream):
    """Stream memory ops the reference's HIP adaptor leaves unimplemented
    (hip_adaptor.cc:319-330): write a flag, then wait on it."""
    h = _malloc(t, 64, N.MEM_HOST)
    flag = _host_view(h, 8, C.c_uint64)
    flag[:] = 0
    d = C.c_void_p()
    assert t.hostGetDevicePointer(C.byref(d), h) == OK
    assert t.streamWriteValue64(stream, d, 41, 0) == OK
    assert t.streamWaitValue64(stream, d, 41, 0) == OK          # flags 0: wait until *addr >= value
    assert t.streamWriteValue64(stream, d.value + 8, 99, 0) == OK
    assert t.streamSynchronize(stream) == OK
    assert flag[0] == 41 and flag[1] == 99
    assert t.streamWaitValue64(None, d, 1, 0) == N.INVALID_ARGUMENT
    assert t.deviceFree(h, N.MEM_HOST, None) == OK


def test_gdr_and_optional_hooks(t):
    p = C.c_void_p()
    assert t.gdrMemAlloc(C.byref(p), 1 << 20, None) == OK and p.value
    assert t.gdrMemFree(p, None) == OK
    assert t.gdrMemAlloc(None, 16, None) == N.INVALID_ARGUMENT
    assert t.getHandleForAddressRange(None, None, 0, 0) == N.NOT_SUPPORTED
    # hooks every built-in adaptor leaves NULL stay NULL (device_plugin_load.cc:66-71)
    assert not t.launchKernel and not t.copyArgsInit and not t.memHandleInit
