"""ctypes view of ``lib/libinfinicore_ops.so``: the framework-side adaptors of the paged operators.

The library does in C++ what the reference's adaptors do between ``infinicore::op::paged_attention_``
and the InfiniOP C API (``src/infinicore/ops/paged_attention/paged_attention_infiniop.cc:18-77``,
``src/infinicore/ops/infiniop_impl.hpp:8-76``): a thread-local LRU cache of operator descriptors per
device keyed by the tensors' metadata, a workspace, and the call, as a plan / run / cleanup triple or
in one step. This module only declares the entry points and turns torch tensors into the plain views
they take; torch provides device memory and the stream, nothing else.
"""
from __future__ import annotations

import ctypes
from ctypes import POINTER, Structure, c_float, c_int, c_size_t, c_ssize_t, c_uint64, c_void_p

import torch

from . import libinfiniop as lib
from .libinfiniop import LIB_DIR, InfiniDevice, InfiniDtype, check_error


class TensorView(Structure):
    """``infinicoreTensorView_t`` (include/infinicore_ops.h)."""

    _fields_ = [("data", c_void_p), ("dtype", c_int), ("ndim", c_size_t), ("shape", POINTER(c_size_t)),
                ("strides", POINTER(c_ssize_t))]


class OpKind:
    PAGED_ATTENTION = 0
    PAGED_ATTENTION_PREFILL = 1
    PAGED_CACHING = 2
    KV_CACHING = 3


_TORCH_TO_INFINI = {
    torch.float16: InfiniDtype.F16,
    torch.bfloat16: InfiniDtype.BF16,
    torch.float32: InfiniDtype.F32,
    torch.int64: InfiniDtype.I64,
    torch.int32: InfiniDtype.I32,
    torch.uint32: InfiniDtype.U32,
    torch.uint8: InfiniDtype.U8,
}


def _open():
    path = LIB_DIR / "libinfinicore_ops.so"
    if not path.is_file():
        raise ImportError(f"{path} not found: build it first (python -m infinicore_amd.build, or __graft_entry__.build())")
    core = ctypes.CDLL(str(path))  # libinfinirt / libinfiniop are loaded (globally) by libinfiniop.py already
    V, P, vp = POINTER(TensorView), c_void_p, c_void_p

    def declare(name, argtypes):
        fn = getattr(core, name)
        fn.argtypes, fn.restype = argtypes, c_int

    declare("infinicoreOpPlanPagedAttention", [POINTER(P), V, V, V, V, V, V, V, c_float])
    declare("infinicoreOpPlanPagedAttentionPrefill", [POINTER(P), V, V, V, V, V, V, V, V, c_float])
    declare("infinicoreOpPlanPagedCaching", [POINTER(P), V, V, V, V, V])
    declare("infinicoreOpPlanKVCaching", [POINTER(P), V, V, V, V, V])
    declare("infinicoreOpRun", [P, vp])
    declare("infinicoreOpCleanup", [POINTER(P)])
    declare("infinicoreOpPlannedWorkspaceSize", [P, POINTER(c_size_t)])
    declare("infinicoreOpPagedAttention", [V, V, V, V, V, V, V, c_float, vp])
    declare("infinicoreOpPagedAttentionPrefill", [V, V, V, V, V, V, V, V, c_float, vp])
    declare("infinicoreOpPagedCaching", [V, V, V, V, V, vp])
    declare("infinicoreOpKVCaching", [V, V, V, V, V, vp])
    declare("infinicoreOpCacheSetCapacity", [c_size_t])
    declare("infinicoreOpCacheStats", [c_int, POINTER(c_size_t), POINTER(c_uint64), POINTER(c_uint64)])
    declare("infinicoreOpCacheClear", [])
    return core


LIBINFINICORE_OPS = _open()


def view(t: torch.Tensor | None, *, contiguous_as_null: bool = False):
    """A ``TensorView`` of a torch CUDA tensor (None stays None). The returned object keeps the extent
    and stride arrays alive; the tensor itself must outlive every use of the view's data pointer."""
    if t is None:
        return None
    if not t.is_cuda:
        raise ValueError("the adaptors work on device tensors only; there is no host fallback")
    ndim = t.dim()
    shape = (c_size_t * max(ndim, 1))(*t.shape)
    strides = None if (contiguous_as_null and t.is_contiguous()) else (c_ssize_t * max(ndim, 1))(*t.stride())
    v = TensorView(c_void_p(t.data_ptr()), _TORCH_TO_INFINI[t.dtype], ndim,
                   ctypes.cast(shape, POINTER(c_size_t)),
                   ctypes.cast(strides, POINTER(c_ssize_t)) if strides is not None else None)
    v._keep = (shape, strides)
    return v


def _refs(views):
    return [ctypes.byref(v) if v is not None else None for v in views]


def _use_device_of(t: torch.Tensor) -> c_void_p:
    index = t.device.index if t.device.index is not None else torch.cuda.current_device()
    lib.set_device(InfiniDevice.AMD, index)
    return c_void_p(torch.cuda.current_stream(index).cuda_stream)


# ---- immediate forms (infinicore::op::paged_attention_ and friends) ----
def paged_attention_(out, q, k_cache, v_cache, block_tables, cache_lens, alibi_slopes=None, scale: float = 1.0):
    stream = _use_device_of(q)
    views = [view(t) for t in (out, q, k_cache, v_cache, block_tables, cache_lens, alibi_slopes)]
    check_error(LIBINFINICORE_OPS.infinicoreOpPagedAttention(*_refs(views), scale, stream), "infinicoreOpPagedAttention")
    return out


def paged_attention_prefill_(out, q, k_cache, v_cache, block_tables, total_kv_lens, cum_seqlens_q, alibi_slopes=None,
                             scale: float = 1.0):
    stream = _use_device_of(q)
    views = [view(t) for t in (out, q, k_cache, v_cache, block_tables, total_kv_lens, cum_seqlens_q, alibi_slopes)]
    check_error(LIBINFINICORE_OPS.infinicoreOpPagedAttentionPrefill(*_refs(views), scale, stream),
                "infinicoreOpPagedAttentionPrefill")
    return out


def paged_caching_(k_cache, v_cache, k, v, slot_mapping):
    stream = _use_device_of(k)
    views = [view(t) for t in (k_cache, v_cache, k, v, slot_mapping)]
    check_error(LIBINFINICORE_OPS.infinicoreOpPagedCaching(*_refs(views), stream), "infinicoreOpPagedCaching")
    return k_cache, v_cache


def kv_caching_(k_cache, v_cache, k, v, past_kv_lengths):
    stream = _use_device_of(k)
    views = [view(t) for t in (k_cache, v_cache, k, v, past_kv_lengths)]
    check_error(LIBINFINICORE_OPS.infinicoreOpKVCaching(*_refs(views), stream), "infinicoreOpKVCaching")
    return k_cache, v_cache


# ---- plan / run / cleanup ----
class PlannedOp:
    """Owns one ``infinicorePlannedOp_t``; keeps the planned-on tensors alive, since the plan holds their
    data pointers (the reference's PlannedMeta holds the tensors themselves)."""

    _PLANNERS = {
        "paged_attention": ("infinicoreOpPlanPagedAttention", 7, True),
        "paged_attention_prefill": ("infinicoreOpPlanPagedAttentionPrefill", 8, True),
        "paged_caching": ("infinicoreOpPlanPagedCaching", 5, False),
        "kv_caching": ("infinicoreOpPlanKVCaching", 5, False),
    }

    def __init__(self, op: str, *tensors, scale: float | None = None):
        name, n_tensors, takes_scale = self._PLANNERS[op]
        if len(tensors) != n_tensors:
            raise TypeError(f"{op} plans on {n_tensors} tensors (the optional one may be None), got {len(tensors)}")
        first = next(t for t in tensors if t is not None)
        _use_device_of(first)
        self._device_index = first.device.index if first.device.index is not None else torch.cuda.current_device()
        self._tensors = tensors
        self._handle = c_void_p()
        views = [view(t) for t in tensors]
        args = [ctypes.byref(self._handle), *_refs(views)] + ([scale if scale is not None else 1.0] if takes_scale else [])
        check_error(getattr(LIBINFINICORE_OPS, name)(*args), name)

    @property
    def workspace_bytes(self) -> int:
        size = c_size_t()
        check_error(LIBINFINICORE_OPS.infinicoreOpPlannedWorkspaceSize(self._handle, ctypes.byref(size)))
        return size.value

    def run(self, stream: torch.cuda.Stream | None = None) -> None:
        s = stream if stream is not None else torch.cuda.current_stream(self._device_index)
        lib.set_device(InfiniDevice.AMD, self._device_index)  # a plan runs on the device it was made on only
        check_error(LIBINFINICORE_OPS.infinicoreOpRun(self._handle, c_void_p(s.cuda_stream)), "infinicoreOpRun")

    def cleanup(self) -> None:
        if self._handle:
            lib.set_device(InfiniDevice.AMD, self._device_index)
            check_error(LIBINFINICORE_OPS.infinicoreOpCleanup(ctypes.byref(self._handle)), "infinicoreOpCleanup")
            self._tensors = ()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.cleanup()


# ---- the calling thread's descriptor caches ----
def cache_set_capacity(capacity: int) -> None:
    check_error(LIBINFINICORE_OPS.infinicoreOpCacheSetCapacity(capacity))


def cache_stats(kind: int) -> tuple[int, int, int]:
    """(entries, hits, misses) of one operator's cache on the current InfiniRT device."""
    entries, hits, misses = c_size_t(), c_uint64(), c_uint64()
    check_error(LIBINFINICORE_OPS.infinicoreOpCacheStats(kind, ctypes.byref(entries), ctypes.byref(hits), ctypes.byref(misses)))
    return entries.value, hits.value, misses.value


def cache_clear() -> None:
    check_error(LIBINFINICORE_OPS.infinicoreOpCacheClear())
