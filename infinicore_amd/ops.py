"""``paged_attention`` / ``paged_attention_prefill`` / ``paged_caching`` on torch CUDA tensors, executed by ``libinfiniop.so``.

Argument order and meaning are those of the reference's Python operators
(``python/infinicore/ops/paged_attention.py:5-40``, ``python/infinicore/ops/paged_attention_prefill.py:5-45``,
``python/infinicore/ops/paged_caching.py:5-21``).
What the reference's C++ adaptor does between that call and the C API
(``src/infinicore/ops/paged_attention/paged_attention_infiniop.cc:16-58``: build tensor descriptors,
fetch or create a cached operator descriptor keyed by the tensors' metadata, allocate a byte
workspace of the size the descriptor asks for, call the operator on the current stream) is done here
with torch providing device memory and the stream.
"""
from __future__ import annotations

import ctypes
from collections import OrderedDict
from ctypes import c_size_t, c_void_p

import torch

from . import libinfiniop as lib
from .libinfiniop import LIBINFINIOP, InfiniDevice, InfiniDtype, check_error

_TORCH_TO_INFINI = {
    torch.float16: InfiniDtype.F16,
    torch.bfloat16: InfiniDtype.BF16,
    torch.float32: InfiniDtype.F32,
    torch.int64: InfiniDtype.I64,
    torch.int32: InfiniDtype.I32,
    torch.uint32: InfiniDtype.U32,
    torch.uint8: InfiniDtype.U8,
    torch.int8: InfiniDtype.I8,
    torch.int16: InfiniDtype.I16,
    torch.uint16: InfiniDtype.U16,
    torch.uint64: InfiniDtype.U64,
}

_PLAN_CACHE_CAPACITY = 100  # the reference keeps a thread-local LRU of 100 descriptors per operator
_handles: dict[int, object] = {}
_plans: "OrderedDict[tuple, _Plan]" = OrderedDict()


def _device_index(t: torch.Tensor) -> int:
    if not t.is_cuda:
        raise ValueError("infinicore_amd.ops works on CUDA (HIP) tensors only; there is no host fallback")
    return t.device.index if t.device.index is not None else torch.cuda.current_device()


def _handle_for(index: int):
    lib.set_device(InfiniDevice.AMD, index)
    if index not in _handles:
        _handles[index] = lib.create_handle()
    return _handles[index]


def _meta(t: torch.Tensor | None):
    return None if t is None else (t.dtype, tuple(t.shape), tuple(t.stride()))


def _describe(t: torch.Tensor):
    return lib.create_tensor_descriptor(tuple(t.shape), tuple(t.stride()), _TORCH_TO_INFINI[t.dtype])


def _ptr(t: torch.Tensor | None):
    return c_void_p(0) if t is None else c_void_p(t.data_ptr())


class _Plan:
    """An operator descriptor plus its workspace; owns both until evicted from the cache. A plan belongs to one
    stream (the stream is part of the cache key): two calls with the same shapes on different streams would
    otherwise write their partial results into the same workspace at the same time."""

    def __init__(self, descriptor, destroy, workspace_bytes: int, device: torch.device):
        self.descriptor = descriptor
        self._destroy = destroy
        self.workspace_bytes = workspace_bytes
        self.workspace = torch.empty(workspace_bytes, dtype=torch.uint8, device=device) if workspace_bytes else None
        self.stream = torch.cuda.current_stream(device)  # the stream of the cache key this plan is stored under

    def close(self):
        if self.workspace is not None:
            # evicted while a kernel on the plan's stream may still be using the workspace: the caching
            # allocator may hand the memory out again only after that stream has passed this point
            self.workspace.record_stream(self.stream)
            self.workspace = None
        if self.descriptor is not None:
            check_error(self._destroy(self.descriptor))
            self.descriptor = None


def _cached_plan(key, make):
    plan = _plans.get(key)
    if plan is not None:
        _plans.move_to_end(key)
        return plan
    plan = make()
    _plans[key] = plan
    if len(_plans) > _PLAN_CACHE_CAPACITY:
        _, old = _plans.popitem(last=False)
        old.close()
    return plan


def clear_plan_cache() -> None:
    while _plans:
        _, plan = _plans.popitem()
        plan.close()


def _stream_key(device_index: int) -> int:
    return int(torch.cuda.current_stream(device_index).cuda_stream)


def _stream_ptr(device_index: int):
    return c_void_p(torch.cuda.current_stream(device_index).cuda_stream)


def paged_attention(q, k_cache, v_cache, block_tables, cache_lens, alibi_slopes=None, scale: float = 1.0, *, out=None):
    """Decode attention of one query token per sequence over a paged KV pool; returns ``out``.

    q [num_seqs, num_heads, head_size]; k_cache / v_cache [num_blocks, num_kv_heads, block_size, d];
    block_tables [num_seqs, max_blocks] and cache_lens [num_seqs] int64/int32/uint32.
    """
    index = _device_index(q)
    if out is None:
        out = torch.empty((*q.shape[:-1], v_cache.shape[-1]), dtype=q.dtype, device=q.device)
    tensors = (out, q, k_cache, v_cache, block_tables, cache_lens)
    key = ("paged_attention", index, _stream_key(index), float(scale), *(_meta(t) for t in tensors), _meta(alibi_slopes))

    def make():
        handle = _handle_for(index)
        descs = [_describe(t) for t in tensors]
        alibi_desc = _describe(alibi_slopes) if alibi_slopes is not None else lib.infiniopTensorDescriptor_t()
        op = lib.infiniopOperatorDescriptor_t()
        try:
            check_error(
                LIBINFINIOP.infiniopCreatePagedAttentionDescriptor(handle, ctypes.byref(op), *descs, alibi_desc, scale),
                "infiniopCreatePagedAttentionDescriptor",
            )
        finally:
            for d in descs:
                lib.destroy_tensor_descriptor(d)
            if alibi_slopes is not None:
                lib.destroy_tensor_descriptor(alibi_desc)
        size = c_size_t(0)
        check_error(LIBINFINIOP.infiniopGetPagedAttentionWorkspaceSize(op, ctypes.byref(size)))
        return _Plan(op, LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor, size.value, q.device)

    plan = _cached_plan(key, make)
    lib.set_device(InfiniDevice.AMD, index)
    check_error(
        LIBINFINIOP.infiniopPagedAttention(
            plan.descriptor, _ptr(plan.workspace), plan.workspace_bytes, _ptr(out), _ptr(q), _ptr(k_cache),
            _ptr(v_cache), _ptr(block_tables), _ptr(cache_lens), _ptr(alibi_slopes), _stream_ptr(index),
        ),
        "infiniopPagedAttention",
    )
    return out


def paged_attention_prefill(q, k_cache, v_cache, block_tables, seq_lens, cum_seq_lens_q, alibi_slopes=None,
                            scale: float = 1.0, *, out=None):
    """Causal attention of each sequence's run of new tokens over its paged K/V; returns ``out``.

    q [total_q_tokens, num_heads, head_size] holds the new tokens of all sequences back to back;
    seq_lens [num_seqs] are the total K/V lengths (history + new), cum_seq_lens_q [num_seqs + 1] the
    prefix sums of the new-token counts; both and block_tables share one index dtype.
    """
    index = _device_index(q)
    if out is None:
        out = torch.empty((*q.shape[:-1], v_cache.shape[-1]), dtype=q.dtype, device=q.device)
    tensors = (out, q, k_cache, v_cache, block_tables, seq_lens, cum_seq_lens_q)
    key = ("paged_attention_prefill", index, _stream_key(index), float(scale), *(_meta(t) for t in tensors), _meta(alibi_slopes))

    def make():
        handle = _handle_for(index)
        descs = [_describe(t) for t in tensors]
        alibi_desc = _describe(alibi_slopes) if alibi_slopes is not None else lib.infiniopTensorDescriptor_t()
        op = lib.infiniopOperatorDescriptor_t()
        try:
            check_error(
                LIBINFINIOP.infiniopCreatePagedAttentionPrefillDescriptor(handle, ctypes.byref(op), *descs, alibi_desc,
                                                                          scale),
                "infiniopCreatePagedAttentionPrefillDescriptor",
            )
        finally:
            for d in descs:
                lib.destroy_tensor_descriptor(d)
            if alibi_slopes is not None:
                lib.destroy_tensor_descriptor(alibi_desc)
        size = c_size_t(0)
        check_error(LIBINFINIOP.infiniopGetPagedAttentionPrefillWorkspaceSize(op, ctypes.byref(size)))
        return _Plan(op, LIBINFINIOP.infiniopDestroyPagedAttentionPrefillDescriptor, size.value, q.device)

    plan = _cached_plan(key, make)
    lib.set_device(InfiniDevice.AMD, index)
    check_error(
        LIBINFINIOP.infiniopPagedAttentionPrefill(
            plan.descriptor, _ptr(plan.workspace), plan.workspace_bytes, _ptr(out), _ptr(q), _ptr(k_cache),
            _ptr(v_cache), _ptr(block_tables), _ptr(seq_lens), _ptr(cum_seq_lens_q), _ptr(alibi_slopes),
            _stream_ptr(index),
        ),
        "infiniopPagedAttentionPrefill",
    )
    return out


def paged_caching(k_cache, v_cache, k, v, slot_mapping):
    """Scatter ``k`` / ``v`` [num_tokens, num_kv_heads, d] into the pools in place; returns the pools."""
    index = _device_index(k)
    tensors = (k_cache, v_cache, k, v, slot_mapping)
    key = ("paged_caching", index, _stream_key(index), *(_meta(t) for t in tensors))

    def make():
        handle = _handle_for(index)
        descs = [_describe(t) for t in tensors]
        op = lib.infiniopOperatorDescriptor_t()
        try:
            check_error(
                LIBINFINIOP.infiniopCreatePagedCachingDescriptor(handle, ctypes.byref(op), *descs),
                "infiniopCreatePagedCachingDescriptor",
            )
        finally:
            for d in descs:
                lib.destroy_tensor_descriptor(d)
        size = c_size_t(0)
        check_error(LIBINFINIOP.infiniopGetPagedCachingWorkspaceSize(op, ctypes.byref(size)))
        return _Plan(op, LIBINFINIOP.infiniopDestroyPagedCachingDescriptor, size.value, k.device)

    plan = _cached_plan(key, make)
    lib.set_device(InfiniDevice.AMD, index)
    check_error(
        LIBINFINIOP.infiniopPagedCaching(
            plan.descriptor, _ptr(plan.workspace), plan.workspace_bytes, _ptr(k_cache), _ptr(v_cache), _ptr(k),
            _ptr(v), _ptr(slot_mapping), _stream_ptr(index),
        ),
        "infiniopPagedCaching",
    )
    return k_cache, v_cache


def rope_paged_caching(k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table,
                       algo: int = lib.RoPEAlgo.GPT_NEOX, *, q=None, q_out=None):
    """Rotate ``k`` [num_tokens, num_kv_heads, head_size] by the rows ``pos_ids`` of the sin / cos tables
    [table_len, head_size / 2] and scatter it, and ``v`` unchanged, into their slots of the paged pools, in one
    launch; returns the pools. The result of the reference's ``rope`` followed by ``paged_caching``
    (python/infinicore/ops/paged_caching.py:5-15 for the scatter's argument order). With ``q``
    [num_tokens, num_heads, head_size] the query is rotated in the same launch, into ``q_out`` (default: in
    place), and the call returns ``(k_cache, v_cache, q_out)``."""
    if q is not None:
        return _rope_qk_paged_caching(q if q_out is None else q_out, q, k_cache, v_cache, k, v, slot_mapping, pos_ids,
                                      sin_table, cos_table, algo)
    index = _device_index(k)
    tensors = (k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table)
    key = ("rope_paged_caching", index, _stream_key(index), int(algo), *(_meta(t) for t in tensors))

    def make():
        handle = _handle_for(index)
        descs = [_describe(t) for t in tensors]
        op = lib.infiniopOperatorDescriptor_t()
        try:
            check_error(
                LIBINFINIOP.infiniopCreateRoPEPagedCachingDescriptor(handle, ctypes.byref(op), *descs, int(algo)),
                "infiniopCreateRoPEPagedCachingDescriptor",
            )
        finally:
            for d in descs:
                lib.destroy_tensor_descriptor(d)
        size = c_size_t(0)
        check_error(LIBINFINIOP.infiniopGetRoPEPagedCachingWorkspaceSize(op, ctypes.byref(size)))
        return _Plan(op, LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor, size.value, k.device)

    plan = _cached_plan(key, make)
    lib.set_device(InfiniDevice.AMD, index)
    check_error(
        LIBINFINIOP.infiniopRoPEPagedCaching(
            plan.descriptor, _ptr(plan.workspace), plan.workspace_bytes, _ptr(k_cache), _ptr(v_cache), _ptr(k),
            _ptr(v), _ptr(slot_mapping), _ptr(pos_ids), _ptr(sin_table), _ptr(cos_table), _stream_ptr(index),
        ),
        "infiniopRoPEPagedCaching",
    )
    return k_cache, v_cache


def _rope_qk_paged_caching(q_out, q, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table, algo):
    index = _device_index(k)
    tensors = (q_out, q, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table)
    key = ("rope_qk_paged_caching", index, _stream_key(index), int(algo), *(_meta(t) for t in tensors))

    def make():
        handle = _handle_for(index)
        descs = [_describe(t) for t in tensors]
        op = lib.infiniopOperatorDescriptor_t()
        try:
            check_error(
                LIBINFINIOP.infiniopCreateRoPEQKPagedCachingDescriptor(handle, ctypes.byref(op), *descs, int(algo)),
                "infiniopCreateRoPEQKPagedCachingDescriptor",
            )
        finally:
            for d in descs:
                lib.destroy_tensor_descriptor(d)
        size = c_size_t(0)
        check_error(LIBINFINIOP.infiniopGetRoPEPagedCachingWorkspaceSize(op, ctypes.byref(size)))
        return _Plan(op, LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor, size.value, k.device)

    plan = _cached_plan(key, make)
    lib.set_device(InfiniDevice.AMD, index)
    check_error(
        LIBINFINIOP.infiniopRoPEQKPagedCaching(
            plan.descriptor, _ptr(plan.workspace), plan.workspace_bytes, *(_ptr(t) for t in tensors), _stream_ptr(index),
        ),
        "infiniopRoPEQKPagedCaching",
    )
    return k_cache, v_cache, q_out


def kv_caching(k_cache, v_cache, k, v, past_kv_lengths):
    """Append ``k`` / ``v`` [batch, num_kv_heads, seq_len, d] to the contiguous caches
    [batch, num_kv_heads, max_seq_len, d] behind the first ``past_kv_lengths[b]`` positions, in place; returns
    the caches (argument order of the reference's infiniopKVCaching, include/infiniop/ops/kv_caching.h:8-29)."""
    index = _device_index(k)
    tensors = (k_cache, v_cache, k, v, past_kv_lengths)
    key = ("kv_caching", index, _stream_key(index), *(_meta(t) for t in tensors))

    def make():
        handle = _handle_for(index)
        descs = [_describe(t) for t in tensors]
        op = lib.infiniopOperatorDescriptor_t()
        try:
            check_error(
                LIBINFINIOP.infiniopCreateKVCachingDescriptor(handle, ctypes.byref(op), *descs),
                "infiniopCreateKVCachingDescriptor",
            )
        finally:
            for d in descs:
                lib.destroy_tensor_descriptor(d)
        size = c_size_t(0)
        check_error(LIBINFINIOP.infiniopGetKVCachingWorkspaceSize(op, ctypes.byref(size)))
        return _Plan(op, LIBINFINIOP.infiniopDestroyKVCachingDescriptor, size.value, k.device)

    plan = _cached_plan(key, make)
    lib.set_device(InfiniDevice.AMD, index)
    check_error(
        LIBINFINIOP.infiniopKVCaching(
            plan.descriptor, _ptr(plan.workspace), plan.workspace_bytes, _ptr(k_cache), _ptr(v_cache), _ptr(k),
            _ptr(v), _ptr(past_kv_lengths), _stream_ptr(index),
        ),
        "infiniopKVCaching",
    )
    return k_cache, v_cache
