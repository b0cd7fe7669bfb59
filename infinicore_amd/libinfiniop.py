"""ctypes view of the C ABI exported by ``lib/libinfinirt.so`` and ``lib/libinfiniop.so``.

Mirrors what the reference's own ctypes harness declares (``test/infiniop/libinfiniop/liboperators.py:58-73``,
``structs.py:11-22``, the ``@OpRegister.operator`` blocks for the two paged operators) so that tests
written against that harness translate line by line. Loading fails loudly when the libraries have not
been built - there is no Python or CPU substitute for them.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_int64, c_size_t, c_uint32, c_uint64, c_void_p
from pathlib import Path

import os

# INFINICORE_AMD_LIB_DIR points at another build of the two libraries (the reference's harness finds
# them through INFINI_ROOT in the same way, test/infiniop/libinfiniop/liboperators.py:20-53).
LIB_DIR = Path(os.environ.get("INFINICORE_AMD_LIB_DIR") or Path(__file__).resolve().parent / "lib")


class InfiniStatus:
    SUCCESS = 0
    INTERNAL_ERROR = 1
    NOT_IMPLEMENTED = 2
    BAD_PARAM = 3
    NULL_POINTER = 4
    DEVICE_TYPE_NOT_SUPPORTED = 5
    DEVICE_NOT_FOUND = 6
    DEVICE_NOT_INITIALIZED = 7
    DEVICE_ARCHITECTURE_NOT_SUPPORTED = 8
    BAD_TENSOR_DTYPE = 10
    BAD_TENSOR_SHAPE = 11
    BAD_TENSOR_STRIDES = 12
    INSUFFICIENT_WORKSPACE = 13


class InfiniDevice:
    CPU = 0
    NVIDIA = 1
    HYGON = 8
    ALI = 10
    AMD = 11
    TYPE_COUNT = 12


class InfiniDtype:
    INVALID = 0
    I8 = 3
    I16 = 4
    I32 = 5
    I64 = 6
    U8 = 7
    U16 = 8
    U32 = 9
    U64 = 10
    F16 = 12
    F32 = 13
    F64 = 14
    BF16 = 19


class RoPEAlgo:
    GPT_J = 0     # pairs are neighbours: (2j, 2j + 1)
    GPT_NEOX = 1  # pairs are half a vector apart: (j, j + d / 2)


class Handle(Structure):
    _fields_ = [("device", c_int), ("device_id", c_int)]


class OpDescriptor(Structure):
    _fields_ = [("device_type", c_int), ("device_id", c_int)]


class TensorDescriptorStruct(Structure):
    _fields_ = []


infiniopHandle_t = POINTER(Handle)
infiniopOperatorDescriptor_t = POINTER(OpDescriptor)
infiniopTensorDescriptor_t = POINTER(TensorDescriptorStruct)


class InfiniStatusError(RuntimeError):
    def __init__(self, status: int, what: str = ""):
        super().__init__(f"InfiniOP call failed with status {status}{(' in ' + what) if what else ''}")
        self.status = status


def check_error(status: int, what: str = "") -> None:
    if status != InfiniStatus.SUCCESS:
        raise InfiniStatusError(status, what)


def _declare(lib, name, argtypes):
    fn = getattr(lib, name)
    fn.argtypes = argtypes
    fn.restype = c_int
    return fn


def _open():
    rt_path, op_path = LIB_DIR / "libinfinirt.so", LIB_DIR / "libinfiniop.so"
    if not rt_path.is_file() or not op_path.is_file():
        raise ImportError(
            f"{rt_path} / {op_path} not found: build them first "
            "(python -m infinicore_amd.build, or __graft_entry__.build())"
        )
    rt = ctypes.CDLL(str(rt_path), mode=ctypes.RTLD_GLOBAL)
    op = ctypes.CDLL(str(op_path))
    vp, T = c_void_p, infiniopTensorDescriptor_t

    # ---- runtime ----
    _declare(rt, "infinirtInit", [])
    _declare(rt, "infinirtGetAllDeviceCount", [POINTER(c_int)])
    _declare(rt, "infinirtGetDeviceCount", [c_int, POINTER(c_int)])
    _declare(rt, "infinirtSetDevice", [c_int, c_int])
    _declare(rt, "infinirtGetDevice", [POINTER(c_int), POINTER(c_int)])
    _declare(rt, "infinirtGetMemInfo", [c_int, c_int, POINTER(c_size_t), POINTER(c_size_t)])
    _declare(rt, "infinirtDeviceSynchronize", [])
    _declare(rt, "infinirtStreamCreate", [POINTER(vp)])
    _declare(rt, "infinirtStreamDestroy", [vp])
    _declare(rt, "infinirtStreamSynchronize", [vp])
    _declare(rt, "infinirtStreamWaitEvent", [vp, vp])
    _declare(rt, "infinirtEventCreate", [POINTER(vp)])
    _declare(rt, "infinirtEventCreateWithFlags", [POINTER(vp), c_uint32])
    _declare(rt, "infinirtEventRecord", [vp, vp])
    _declare(rt, "infinirtEventQuery", [vp, POINTER(c_int)])
    _declare(rt, "infinirtEventSynchronize", [vp])
    _declare(rt, "infinirtEventDestroy", [vp])
    _declare(rt, "infinirtEventElapsedTime", [POINTER(c_float), vp, vp])
    _declare(rt, "infinirtMalloc", [POINTER(vp), c_size_t])
    _declare(rt, "infinirtMallocHost", [POINTER(vp), c_size_t])
    _declare(rt, "infinirtFree", [vp])
    _declare(rt, "infinirtFreeHost", [vp])
    _declare(rt, "infinirtMemcpy", [vp, vp, c_size_t, c_int])
    _declare(rt, "infinirtMemcpyAsync", [vp, vp, c_size_t, c_int, vp])
    _declare(rt, "infinirtMallocAsync", [POINTER(vp), c_size_t, vp])
    _declare(rt, "infinirtFreeAsync", [vp, vp])
    _declare(rt, "infinirtMemset", [vp, c_int, c_size_t])
    _declare(rt, "infinirtMemsetAsync", [vp, c_int, c_size_t, vp])
    _declare(rt, "infinirtStreamBeginCapture", [vp, c_int])
    _declare(rt, "infinirtStreamEndCapture", [vp, POINTER(vp)])
    _declare(rt, "infinirtGraphDestroy", [vp])
    _declare(rt, "infinirtGraphInstantiate", [POINTER(vp), vp, POINTER(vp), ctypes.c_char_p, c_size_t])
    _declare(rt, "infinirtGraphExecDestroy", [vp])
    _declare(rt, "infinirtGraphLuanch", [vp, vp])

    # ---- operator library: context objects ----
    _declare(op, "infiniopCreateHandle", [POINTER(infiniopHandle_t)])
    _declare(op, "infiniopDestroyHandle", [infiniopHandle_t])
    _declare(op, "infiniopCreateTensorDescriptor", [POINTER(T), c_uint64, POINTER(c_uint64), POINTER(c_int64), c_int])
    _declare(op, "infiniopDestroyTensorDescriptor", [T])
    _declare(op, "infiniopGetDescriptorDeviceType", [infiniopOperatorDescriptor_t, POINTER(c_int)])
    _declare(op, "infiniopGetDescriptorDeviceId", [infiniopOperatorDescriptor_t, POINTER(c_int)])

    # ---- paged_attention ----
    D = infiniopOperatorDescriptor_t
    _declare(op, "infiniopCreatePagedAttentionDescriptor", [infiniopHandle_t, POINTER(D), T, T, T, T, T, T, T, c_float])
    _declare(op, "infiniopGetPagedAttentionWorkspaceSize", [D, POINTER(c_size_t)])
    _declare(op, "infiniopPagedAttention", [D, vp, c_size_t, vp, vp, vp, vp, vp, vp, vp, vp])
    _declare(op, "infiniopPagedAttentionNoAlloc", [D, vp, vp, vp, vp, vp, vp, vp, vp])
    _declare(op, "infiniopDestroyPagedAttentionDescriptor", [D])

    # ---- paged_attention_prefill ----
    _declare(op, "infiniopCreatePagedAttentionPrefillDescriptor", [infiniopHandle_t, POINTER(D), T, T, T, T, T, T, T, T, c_float])
    _declare(op, "infiniopGetPagedAttentionPrefillWorkspaceSize", [D, POINTER(c_size_t)])
    _declare(op, "infiniopPagedAttentionPrefill", [D, vp, c_size_t, vp, vp, vp, vp, vp, vp, vp, vp, vp])
    _declare(op, "infiniopDestroyPagedAttentionPrefillDescriptor", [D])

    # ---- paged_caching ----
    _declare(op, "infiniopCreatePagedCachingDescriptor", [infiniopHandle_t, POINTER(D), T, T, T, T, T])
    _declare(op, "infiniopGetPagedCachingWorkspaceSize", [D, POINTER(c_size_t)])
    _declare(op, "infiniopPagedCaching", [D, vp, c_size_t, vp, vp, vp, vp, vp, vp])
    _declare(op, "infiniopDestroyPagedCachingDescriptor", [D])
    _declare(op, "infiniopCreateRoPEPagedCachingDescriptor", [infiniopHandle_t, POINTER(D), T, T, T, T, T, T, T, T, c_int])
    _declare(op, "infiniopGetRoPEPagedCachingWorkspaceSize", [D, POINTER(c_size_t)])
    _declare(op, "infiniopRoPEPagedCaching", [D, vp, c_size_t, vp, vp, vp, vp, vp, vp, vp, vp, vp])
    _declare(op, "infiniopDestroyRoPEPagedCachingDescriptor", [D])
    _declare(op, "infiniopCreateRoPEQKPagedCachingDescriptor", [infiniopHandle_t, POINTER(D)] + [T] * 10 + [c_int])
    _declare(op, "infiniopRoPEQKPagedCaching", [D, vp, c_size_t] + [vp] * 11)
    _declare(op, "infiniopCreateKVCachingDescriptor", [infiniopHandle_t, POINTER(D), T, T, T, T, T])
    _declare(op, "infiniopGetKVCachingWorkspaceSize", [D, POINTER(c_size_t)])
    _declare(op, "infiniopKVCaching", [D, vp, c_size_t, vp, vp, vp, vp, vp, vp])
    _declare(op, "infiniopDestroyKVCachingDescriptor", [D])
    return rt, op


LIBINFINIRT, LIBINFINIOP = _open()


def create_tensor_descriptor(shape, strides, dtype: int):
    """``strides`` in elements, or None for a C-contiguous tensor. Caller destroys the result."""
    ndim = len(shape)
    c_shape = (c_uint64 * ndim)(*shape)
    c_strides = (c_int64 * ndim)(*strides) if strides is not None else None
    desc = infiniopTensorDescriptor_t()
    check_error(
        LIBINFINIOP.infiniopCreateTensorDescriptor(ctypes.byref(desc), ndim, c_shape, c_strides, dtype),
        "infiniopCreateTensorDescriptor",
    )
    return desc


def destroy_tensor_descriptor(desc) -> None:
    check_error(LIBINFINIOP.infiniopDestroyTensorDescriptor(desc), "infiniopDestroyTensorDescriptor")


def set_device(device: int, device_id: int = 0) -> None:
    check_error(LIBINFINIRT.infinirtSetDevice(device, device_id), "infinirtSetDevice")


def create_handle():
    handle = infiniopHandle_t()
    check_error(LIBINFINIOP.infiniopCreateHandle(ctypes.byref(handle)), "infiniopCreateHandle")
    return handle


def destroy_handle(handle) -> None:
    check_error(LIBINFINIOP.infiniopDestroyHandle(handle), "infiniopDestroyHandle")
