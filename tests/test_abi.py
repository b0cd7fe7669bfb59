"""The C-ABI libraries load and export every symbol the public headers declare (no GPU needed)."""
import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADERS = sorted((ROOT / "include").rglob("*.h"))
PROTOTYPE = re.compile(r"__INFINI_C\s+__export\s+infiniStatus_t\s+(\w+)\s*\(")


def declared_symbols():
    names = []
    for header in HEADERS:
        names += [(header.relative_to(ROOT).as_posix(), n) for n in PROTOTYPE.findall(header.read_text())]
    return names


def test_headers_declare_the_expected_entry_points():
    names = {n for _, n in declared_symbols()}
    for required in (
        "infiniopCreatePagedAttentionDescriptor", "infiniopGetPagedAttentionWorkspaceSize", "infiniopPagedAttention",
        "infiniopDestroyPagedAttentionDescriptor", "infiniopCreatePagedAttentionPrefillDescriptor",
        "infiniopGetPagedAttentionPrefillWorkspaceSize", "infiniopPagedAttentionPrefill",
        "infiniopDestroyPagedAttentionPrefillDescriptor", "infiniopCreatePagedCachingDescriptor",
        "infiniopGetPagedCachingWorkspaceSize", "infiniopPagedCaching", "infiniopDestroyPagedCachingDescriptor",
        "infiniopCreateKVCachingDescriptor", "infiniopGetKVCachingWorkspaceSize", "infiniopKVCaching",
        "infiniopDestroyKVCachingDescriptor",
        "infiniopCreateHandle", "infiniopDestroyHandle", "infiniopCreateTensorDescriptor",
        "infiniopDestroyTensorDescriptor", "infinirtSetDevice", "infinirtMalloc", "infinirtStreamCreate",
    ):
        assert required in names


@pytest.mark.parametrize("header,symbol", declared_symbols())
def test_symbol_is_exported(lib, header, symbol):
    if symbol.startswith("infinicoreOp"):
        from infinicore_amd import libinfinicore_ops

        owner = libinfinicore_ops.LIBINFINICORE_OPS
    else:
        owner = lib.LIBINFINIRT if symbol.startswith("infinirt") else lib.LIBINFINIOP
    assert hasattr(owner, symbol), f"{symbol} (declared in {header}) is not exported"


def test_headers_compile_as_c():
    import subprocess

    for header in ("infiniop.h", "infinirt.h", "infinicore_ops.h"):
        subprocess.run(["gcc", "-fsyntax-only", "-x", "c", "-I", str(ROOT / "include"), str(ROOT / "include" / header)],
                       check=True)


def test_enum_values_match_the_reference_abi(lib):
    # include/infinicore.h:20-76 of the reference; AMD is the appended device
    assert lib.InfiniStatus.INSUFFICIENT_WORKSPACE == 13 and lib.InfiniStatus.BAD_TENSOR_STRIDES == 12
    assert lib.InfiniDtype.F16 == 12 and lib.InfiniDtype.BF16 == 19 and lib.InfiniDtype.I64 == 6
    assert lib.InfiniDevice.ALI == 10 and lib.InfiniDevice.AMD == 11 and lib.InfiniDevice.TYPE_COUNT == 12


def test_runtime_on_a_host_without_gpu_or_with(lib):
    """CPU device bookkeeping works everywhere; the AMD device count is just reported."""
    counts = (ctypes.c_int * lib.InfiniDevice.TYPE_COUNT)()
    assert lib.LIBINFINIRT.infinirtGetAllDeviceCount(counts) == 0
    assert counts[lib.InfiniDevice.CPU] == 1
    assert counts[lib.InfiniDevice.NVIDIA] == 0
    assert lib.LIBINFINIRT.infinirtGetAllDeviceCount(None) == lib.InfiniStatus.NULL_POINTER
    # a device type without a backend
    assert lib.LIBINFINIRT.infinirtSetDevice(lib.InfiniDevice.NVIDIA, 0) == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    # an AMD device id that cannot exist
    assert lib.LIBINFINIRT.infinirtSetDevice(lib.InfiniDevice.AMD, 4096) == lib.InfiniStatus.DEVICE_NOT_FOUND
    # CPU: current device is per thread and starts as CPU:0
    assert lib.LIBINFINIRT.infinirtSetDevice(lib.InfiniDevice.CPU, 0) == 0
    dev, idx = ctypes.c_int(-1), ctypes.c_int(-1)
    assert lib.LIBINFINIRT.infinirtGetDevice(ctypes.byref(dev), ctypes.byref(idx)) == 0
    assert (dev.value, idx.value) == (lib.InfiniDevice.CPU, 0)
    assert lib.LIBINFINIRT.infinirtGetDevice(None, None) == lib.InfiniStatus.NULL_POINTER


def test_host_backend_memory_and_events(lib):
    rt = lib.LIBINFINIRT
    assert rt.infinirtSetDevice(lib.InfiniDevice.CPU, 0) == 0
    a, b = ctypes.c_void_p(), ctypes.c_void_p()
    assert rt.infinirtMalloc(ctypes.byref(a), 64) == 0 and rt.infinirtMallocHost(ctypes.byref(b), 64) == 0
    assert rt.infinirtMemset(a, 0x5A, 64) == 0
    assert rt.infinirtMemcpy(b, a, 64, 0) == 0
    assert bytes((ctypes.c_char * 64).from_address(b.value)) == b"\x5a" * 64
    e0, e1 = ctypes.c_void_p(), ctypes.c_void_p()
    assert rt.infinirtEventCreate(ctypes.byref(e0)) == 0 and rt.infinirtEventCreate(ctypes.byref(e1)) == 0
    assert rt.infinirtEventRecord(e0, None) == 0 and rt.infinirtEventRecord(e1, None) == 0
    ms = ctypes.c_float(-1)
    assert rt.infinirtEventElapsedTime(ctypes.byref(ms), e0, e1) == 0 and ms.value >= 0
    status = ctypes.c_int(-1)
    assert rt.infinirtEventQuery(e0, ctypes.byref(status)) == 0 and status.value == 0
    assert rt.infinirtEventDestroy(e0) == 0 and rt.infinirtEventDestroy(e1) == 0
    assert rt.infinirtFree(a) == 0 and rt.infinirtFreeHost(b) == 0
    assert rt.infinirtMalloc(None, 8) == lib.InfiniStatus.NULL_POINTER


def test_cpu_handle_and_unsupported_device_for_the_paged_ops(lib):
    """A CPU handle can be created, but the paged operators have no CPU backend - exactly as in the
    reference (src/infiniop/ops/paged_attention/operator.cc:42-69 has no CPU case)."""
    assert lib.LIBINFINIRT.infinirtSetDevice(lib.InfiniDevice.CPU, 0) == 0
    handle = lib.create_handle()
    assert handle.contents.device == lib.InfiniDevice.CPU
    shape = (2, 4, 128)
    t = lib.create_tensor_descriptor(shape, None, lib.InfiniDtype.F16)
    op = lib.infiniopOperatorDescriptor_t()
    status = lib.LIBINFINIOP.infiniopCreatePagedAttentionDescriptor(handle, ctypes.byref(op), t, t, t, t, t, t, None, 1.0)
    assert status == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    status = lib.LIBINFINIOP.infiniopCreatePagedCachingDescriptor(handle, ctypes.byref(op), t, t, t, t, t)
    assert status == lib.InfiniStatus.DEVICE_TYPE_NOT_SUPPORTED
    lib.destroy_tensor_descriptor(t)
    lib.destroy_handle(handle)
    assert lib.LIBINFINIOP.infiniopCreateHandle(None) == lib.InfiniStatus.NULL_POINTER
