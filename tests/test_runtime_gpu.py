"""InfiniRT on the AMD device: memory, copies, streams, events - the calls the operators' callers use
(reference smoke test: src/infinirt-test/)."""
import ctypes

import pytest

pytestmark = pytest.mark.gpu


def test_device_memory_streams_and_events(lib):
    rt, AMD = lib.LIBINFINIRT, lib.InfiniDevice.AMD
    count = ctypes.c_int(0)
    assert rt.infinirtGetDeviceCount(AMD, ctypes.byref(count)) == 0 and count.value >= 1
    assert rt.infinirtSetDevice(AMD, 0) == 0
    dev, idx = ctypes.c_int(-1), ctypes.c_int(-1)
    assert rt.infinirtGetDevice(ctypes.byref(dev), ctypes.byref(idx)) == 0 and (dev.value, idx.value) == (AMD, 0)
    free_b, total_b = ctypes.c_size_t(0), ctypes.c_size_t(0)
    assert rt.infinirtGetMemInfo(AMD, 0, ctypes.byref(free_b), ctypes.byref(total_b)) == 0
    assert total_b.value > 100 * 2 ** 30 and free_b.value <= total_b.value  # 288 GB part

    n = 1 << 20
    d_a, d_b, h = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    assert rt.infinirtMalloc(ctypes.byref(d_a), n) == 0 and rt.infinirtMalloc(ctypes.byref(d_b), n) == 0
    assert rt.infinirtMallocHost(ctypes.byref(h), n) == 0
    host = (ctypes.c_ubyte * n).from_address(h.value)
    for i in range(0, n, 4097):
        host[i] = i % 251
    stream, e0, e1 = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    assert rt.infinirtStreamCreate(ctypes.byref(stream)) == 0
    assert rt.infinirtEventCreate(ctypes.byref(e0)) == 0 and rt.infinirtEventCreateWithFlags(ctypes.byref(e1), 0) == 0
    assert rt.infinirtEventRecord(e0, stream) == 0
    assert rt.infinirtMemcpyAsync(d_a, h, n, 1, stream) == 0          # H2D
    assert rt.infinirtMemcpyAsync(d_b, d_a, n, 3, stream) == 0        # D2D
    assert rt.infinirtMemsetAsync(d_a, 0, n, stream) == 0
    assert rt.infinirtEventRecord(e1, stream) == 0
    assert rt.infinirtStreamWaitEvent(stream, e1) == 0
    assert rt.infinirtStreamSynchronize(stream) == 0
    status = ctypes.c_int(-1)
    assert rt.infinirtEventQuery(e1, ctypes.byref(status)) == 0 and status.value == 0
    ms = ctypes.c_float(-1)
    assert rt.infinirtEventElapsedTime(ctypes.byref(ms), e0, e1) == 0 and ms.value >= 0
    back = (ctypes.c_ubyte * n)()
    assert rt.infinirtMemcpy(back, d_b, n, 2) == 0                    # D2H
    assert all(back[i] == i % 251 for i in range(0, n, 4097))
    assert rt.infinirtMemcpy(back, d_a, n, 2) == 0
    assert not any(back[i] for i in range(0, n, 4097))
    assert rt.infinirtDeviceSynchronize() == 0
    for ev in (e0, e1):
        assert rt.infinirtEventDestroy(ev) == 0
    assert rt.infinirtStreamDestroy(stream) == 0
    assert rt.infinirtFree(d_a) == 0 and rt.infinirtFree(d_b) == 0 and rt.infinirtFreeHost(h) == 0


def test_handle_records_the_current_device(lib, gpu_handle):
    assert gpu_handle.contents.device == lib.InfiniDevice.AMD and gpu_handle.contents.device_id == 0
