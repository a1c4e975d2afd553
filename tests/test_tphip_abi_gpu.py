"""The utility entries of the tphip C ABI, one by one, on a real GPU: devices and
pointers, memory, streams and events, IPC handles. (The copy entries have their
own file; the channels use all of these indirectly.)"""
import ctypes
import re

import numpy as np
import pytest

from tensorpipe_amd import _native

pytestmark = pytest.mark.gpu

vp = ctypes.c_void_p


@pytest.fixture(scope="module")
def lib():
    lib = _native.tphip()
    lib.tphip_stream_on_complete.argtypes = [
        ctypes.c_int, vp, ctypes.CFUNCTYPE(None, vp, ctypes.c_int), vp]
    return lib


def _malloc(lib, n):
    p = vp()
    _native.check(lib.tphip_malloc(0, n, ctypes.byref(p)))
    return p


def test_devices_and_uuid(lib):
    count = ctypes.c_int(-1)
    _native.check(lib.tphip_device_count(ctypes.byref(count)))
    assert count.value >= 1
    out = ctypes.create_string_buffer(37)
    _native.check(lib.tphip_device_uuid(0, out))
    # 8-4-4-4-12 hex digits (tensorpipe/common/cuda.h:293-321 prints NVML's the same way)
    assert re.fullmatch(r"[0-9a-f]{8}-[0-9a-f]{4}-[0-9a-f]{4}-[0-9a-f]{4}-[0-9a-f]{12}", out.value.decode())
    again = ctypes.create_string_buffer(37)
    _native.check(lib.tphip_device_uuid(0, again))
    assert again.value == out.value
    assert lib.tphip_device_uuid(0, None) == -1
    assert lib.tphip_device_uuid(count.value + 7, out) != 0


def test_pointer_queries(lib):
    n = 1 << 20
    p = _malloc(lib, n)
    dev, is_host = ctypes.c_int(-5), ctypes.c_int(-5)
    _native.check(lib.tphip_device_for_ptr(vp(p.value + 12345), ctypes.byref(dev), ctypes.byref(is_host)))
    assert (dev.value, is_host.value) == (0, 0)
    base, size = vp(), ctypes.c_size_t()
    _native.check(lib.tphip_mem_base(vp(p.value + 12345), ctypes.byref(base), ctypes.byref(size)))
    assert base.value == p.value and size.value >= n
    ident, other_ident = ctypes.c_uint64(), ctypes.c_uint64()
    _native.check(lib.tphip_mem_buffer_id(vp(p.value + 5), ctypes.byref(ident)))
    q = _malloc(lib, n)
    _native.check(lib.tphip_mem_buffer_id(q, ctypes.byref(other_ident)))
    assert ident.value != 0 and other_ident.value != 0 and ident.value != other_ident.value
    # an address that is freed and handed out again is a new allocation
    seen = {ident.value, other_ident.value}
    _native.check(lib.tphip_free(0, q))
    r = _malloc(lib, n)
    fresh = ctypes.c_uint64()
    _native.check(lib.tphip_mem_buffer_id(r, ctypes.byref(fresh)))
    assert fresh.value not in seen
    # pinned host memory: a host allocation that the device can address
    host, devp = vp(), vp()
    _native.check(lib.tphip_host_alloc(0, 4096, ctypes.byref(host), ctypes.byref(devp)))
    _native.check(lib.tphip_device_for_ptr(host, ctypes.byref(dev), ctypes.byref(is_host)))
    assert is_host.value == 1
    # ordinary host memory is unknown to the runtime
    plain = np.zeros(64, np.uint8)
    rc = lib.tphip_device_for_ptr(vp(plain.ctypes.data), ctypes.byref(dev), ctypes.byref(is_host))
    assert rc != 0 or dev.value == -1 or is_host.value == 1
    _native.check(lib.tphip_host_free(host))
    _native.check(lib.tphip_free(0, r))
    _native.check(lib.tphip_free(0, p))


def test_pointer_queries_from_a_fresh_thread(lib):
    # tensorpipe/test/common/cuda_test.cc:33-62 (DeviceForPointer), on the one device there is: a
    # thread that has made no GPU call yet asks where a pointer of another thread lives
    import threading

    p = _malloc(lib, 1024)
    seen = {}

    def ask():
        dev, is_host = ctypes.c_int(-5), ctypes.c_int(-5)
        seen["rc"] = lib.tphip_device_for_ptr(vp(p.value + 100), ctypes.byref(dev), ctypes.byref(is_host))
        seen["dev"], seen["is_host"] = dev.value, is_host.value
        ident = ctypes.c_uint64()
        seen["rc_id"] = lib.tphip_mem_buffer_id(p, ctypes.byref(ident))
        seen["id"] = ident.value

    t = threading.Thread(target=ask)
    t.start()
    t.join()
    here = ctypes.c_uint64()
    _native.check(lib.tphip_mem_buffer_id(p, ctypes.byref(here)))
    assert seen == {"rc": 0, "dev": 0, "is_host": 0, "rc_id": 0, "id": here.value}
    _native.check(lib.tphip_free(0, p))


def test_pinned_host_slab_is_visible_to_both_sides(lib):
    n = 1 << 16
    host, devp = vp(), vp()
    _native.check(lib.tphip_host_alloc(0, n, ctypes.byref(host), ctypes.byref(devp)))
    view = np.ctypeslib.as_array(ctypes.cast(host, ctypes.POINTER(ctypes.c_uint8)), shape=(n,))
    view[:] = np.arange(n, dtype=np.uint32).astype(np.uint8)
    d = _malloc(lib, n)
    _native.check(lib.tphip_copy(0, d, devp, n, None))          # host slab -> device, by the kernel
    _native.check(lib.tphip_fill(0, devp, 0, n, None))           # device writes the host slab
    _native.check(lib.tphip_stream_sync(0, None))
    assert (view == 0).all()
    _native.check(lib.tphip_copy(0, devp, d, n, None))          # and back
    _native.check(lib.tphip_stream_sync(0, None))
    assert (view == np.arange(n, dtype=np.uint32).astype(np.uint8)).all()
    _native.check(lib.tphip_free(0, d))
    _native.check(lib.tphip_host_free(host))


def test_streams_and_events(lib):
    n = 4096
    buf = _malloc(lib, n)
    s1, s2 = vp(), vp()
    _native.check(lib.tphip_stream_create(0, ctypes.byref(s1)))
    _native.check(lib.tphip_stream_create(0, ctypes.byref(s2)))
    done = ctypes.c_int(-1)
    _native.check(lib.tphip_stream_query(0, s1, ctypes.byref(done)))
    assert done.value == 1  # nothing enqueued yet
    ev = vp()
    _native.check(lib.tphip_event_create(0, 0, ctypes.byref(ev)))
    _native.check(lib.tphip_event_query(0, ev, ctypes.byref(done)))
    assert done.value == 1  # never recorded
    # s1: slow kernel scribbling over buf, then the fill that must win; s2 waits for s1's event
    # before it copies (ReceiverWaitsForStartEvent, channel_test_cuda.cc:19-94, at this level)
    out = _malloc(lib, n)
    _native.check(lib.tphip_test_slow_kernel(0, buf, n, s1))
    _native.check(lib.tphip_fill(0, buf, 0x42, n, s1))
    _native.check(lib.tphip_event_record(0, ev, s1))
    _native.check(lib.tphip_stream_query(0, s1, ctypes.byref(done)))
    assert done.value == 0  # the slow kernel takes tens of milliseconds
    _native.check(lib.tphip_event_query(0, ev, ctypes.byref(done)))
    assert done.value == 0
    _native.check(lib.tphip_stream_wait_event(0, s2, ev))
    _native.check(lib.tphip_copy(0, out, buf, n, s2))
    _native.check(lib.tphip_stream_sync(0, s2))
    host = np.zeros(n, np.uint8)
    _native.check(lib.tphip_memcpy_async(0, vp(host.ctypes.data), out, n, s2))
    _native.check(lib.tphip_stream_sync(0, s2))
    assert (host == 0x42).all()
    _native.check(lib.tphip_event_sync(0, ev))
    _native.check(lib.tphip_event_query(0, ev, ctypes.byref(done)))
    assert done.value == 1
    # timed events bracket a copy
    t0, t1 = vp(), vp()
    _native.check(lib.tphip_event_create_timed(0, ctypes.byref(t0)))
    _native.check(lib.tphip_event_create_timed(0, ctypes.byref(t1)))
    big = 64 << 20
    a, b = _malloc(lib, big), _malloc(lib, big)
    _native.check(lib.tphip_event_record(0, t0, s1))
    _native.check(lib.tphip_copy(0, b, a, big, s1))
    _native.check(lib.tphip_event_record(0, t1, s1))
    _native.check(lib.tphip_event_sync(0, t1))
    ms = ctypes.c_float(-1)
    _native.check(lib.tphip_event_elapsed_ms(t0, t1, ctypes.byref(ms)))
    assert 0.005 < ms.value < 5.0  # 64 MiB take about 0.02 ms
    for e in (ev, t0, t1):
        _native.check(lib.tphip_event_destroy(0, e))
    for s in (s1, s2):
        _native.check(lib.tphip_stream_destroy(0, s))
    for p in (buf, out, a, b):
        _native.check(lib.tphip_free(0, p))


def test_ipc_handles(lib):
    n = 1 << 20
    p = _malloc(lib, n)
    handle = ctypes.create_string_buffer(64)
    _native.check(lib.tphip_ipc_mem_export(0, p, handle))
    assert any(handle.raw)  # something was written
    # the tail of the 64 bytes is not part of the handle's meaning and changes from one export of
    # the same allocation to the next: nothing may key on the handle bytes
    again = ctypes.create_string_buffer(64)
    _native.check(lib.tphip_ipc_mem_export(0, p, again))
    assert again.raw[:32] == handle.raw[:32]
    # events: exporting may be refused by the runtime (it is on the deployment this was built on,
    # which is why the channels synchronise through the host); either way the call answers
    ev = vp()
    _native.check(lib.tphip_event_create(0, 1, ctypes.byref(ev)))
    ehandle = ctypes.create_string_buffer(64)
    rc = lib.tphip_ipc_event_export(0, ev, ehandle)
    assert rc == 0 or lib.tphip_strerror(rc)
    _native.check(lib.tphip_event_destroy(0, ev))
    _native.check(lib.tphip_free(0, p))
