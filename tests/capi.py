"""Helpers that drive the operators through the raw C ABI the way the reference's ctypes tests do
(test/infiniop/paged_attention.py:185-263, test/infiniop/paged_caching.py:160-232): build tensor
descriptors, create the operator descriptor, query the workspace, destroy the tensor descriptors
BEFORE running (the operator must own its metadata), run on the NULL stream, synchronise."""
from __future__ import annotations

import ctypes
from ctypes import c_size_t, c_void_p

import torch

from infinicore_amd import libinfiniop as L

TORCH_TO_INFINI = {
    torch.float16: L.InfiniDtype.F16,
    torch.bfloat16: L.InfiniDtype.BF16,
    torch.float32: L.InfiniDtype.F32,
    torch.int64: L.InfiniDtype.I64,
    torch.int32: L.InfiniDtype.I32,
    torch.uint32: L.InfiniDtype.U32,
    torch.int8: L.InfiniDtype.I8,
    torch.uint8: L.InfiniDtype.U8,
    torch.int16: L.InfiniDtype.I16,
    torch.uint16: L.InfiniDtype.U16,
    torch.uint64: L.InfiniDtype.U64,
}


def describe(t: torch.Tensor, dtype=None):
    return L.create_tensor_descriptor(tuple(t.shape), tuple(t.stride()), dtype or TORCH_TO_INFINI[t.dtype])


def ptr(t):
    return c_void_p(0) if t is None else c_void_p(t.data_ptr())


def create_paged_attention(handle, out, q, k_cache, v_cache, block_tables, seq_lens, alibi, scale):
    """Returns (status, descriptor). Tensor descriptors are destroyed before returning."""
    descs = [describe(t) for t in (out, q, k_cache, v_cache, block_tables, seq_lens)]
    alibi_desc = describe(alibi) if alibi is not None else L.infiniopTensorDescriptor_t()
    op = L.infiniopOperatorDescriptor_t()
    status = L.LIBINFINIOP.infiniopCreatePagedAttentionDescriptor(handle, ctypes.byref(op), *descs, alibi_desc, scale)
    for d in descs:
        L.destroy_tensor_descriptor(d)
    if alibi is not None:
        L.destroy_tensor_descriptor(alibi_desc)
    return status, op


def workspace_size_attention(op) -> int:
    size = c_size_t(0)
    L.check_error(L.LIBINFINIOP.infiniopGetPagedAttentionWorkspaceSize(op, ctypes.byref(size)))
    return size.value


def run_paged_attention(handle, q, k_cache, v_cache, block_tables, seq_lens, scale, alibi=None, out=None,
                        stream=None, workspace_fill=1):
    """Full create / query / run / destroy cycle on device tensors; returns ``out``."""
    if out is None:
        out = torch.zeros((*q.shape[:-1], v_cache.shape[-1]), dtype=q.dtype, device=q.device)
    status, op = create_paged_attention(handle, out, q, k_cache, v_cache, block_tables, seq_lens, alibi, scale)
    L.check_error(status, "infiniopCreatePagedAttentionDescriptor")
    size = workspace_size_attention(op)
    # the reference harness hands over a workspace of ones (TestWorkspace); content must not matter
    workspace = torch.full((max(size, 1),), workspace_fill, dtype=torch.uint8, device=q.device)
    torch.cuda.synchronize()
    L.check_error(
        L.LIBINFINIOP.infiniopPagedAttention(op, ptr(workspace), size, ptr(out), ptr(q), ptr(k_cache), ptr(v_cache),
                                             ptr(block_tables), ptr(seq_lens), ptr(alibi), c_void_p(stream or 0)),
        "infiniopPagedAttention",
    )
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))
    return out


def create_paged_attention_prefill(handle, out, q, k_cache, v_cache, block_tables, seq_lens, cum_seq_lens_q, alibi,
                                   scale):
    """Returns (status, descriptor). Tensor descriptors are destroyed before returning."""
    descs = [describe(t) for t in (out, q, k_cache, v_cache, block_tables, seq_lens, cum_seq_lens_q)]
    alibi_desc = describe(alibi) if alibi is not None else L.infiniopTensorDescriptor_t()
    op = L.infiniopOperatorDescriptor_t()
    status = L.LIBINFINIOP.infiniopCreatePagedAttentionPrefillDescriptor(handle, ctypes.byref(op), *descs, alibi_desc,
                                                                         scale)
    for d in descs:
        L.destroy_tensor_descriptor(d)
    if alibi is not None:
        L.destroy_tensor_descriptor(alibi_desc)
    return status, op


def run_paged_attention_prefill(handle, q, k_cache, v_cache, block_tables, seq_lens, cum_seq_lens_q, scale, alibi=None,
                                out=None, stream=None):
    """Full create / query / run / destroy cycle on device tensors (the sequence of calls of
    test/infiniop/paged_attention_prefill.py:259-310); returns ``out``."""
    if out is None:
        out = torch.zeros((*q.shape[:-1], v_cache.shape[-1]), dtype=q.dtype, device=q.device)
    status, op = create_paged_attention_prefill(handle, out, q, k_cache, v_cache, block_tables, seq_lens,
                                                cum_seq_lens_q, alibi, scale)
    L.check_error(status, "infiniopCreatePagedAttentionPrefillDescriptor")
    size = c_size_t(123)
    L.check_error(L.LIBINFINIOP.infiniopGetPagedAttentionPrefillWorkspaceSize(op, ctypes.byref(size)))
    workspace = torch.full((max(size.value, 1),), 1, dtype=torch.uint8, device=q.device)
    torch.cuda.synchronize()
    L.check_error(
        L.LIBINFINIOP.infiniopPagedAttentionPrefill(op, ptr(workspace), size.value, ptr(out), ptr(q), ptr(k_cache),
                                                    ptr(v_cache), ptr(block_tables), ptr(seq_lens),
                                                    ptr(cum_seq_lens_q), ptr(alibi), c_void_p(stream or 0)),
        "infiniopPagedAttentionPrefill",
    )
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionPrefillDescriptor(op))
    return out


def create_paged_caching(handle, k_cache, v_cache, k, v, slot_mapping):
    descs = [describe(t) for t in (k_cache, v_cache, k, v, slot_mapping)]
    op = L.infiniopOperatorDescriptor_t()
    status = L.LIBINFINIOP.infiniopCreatePagedCachingDescriptor(handle, ctypes.byref(op), *descs)
    for d in descs:
        L.destroy_tensor_descriptor(d)
    return status, op


def run_paged_caching(handle, k_cache, v_cache, k, v, slot_mapping, stream=None):
    """In place on the device pools; returns them."""
    status, op = create_paged_caching(handle, k_cache, v_cache, k, v, slot_mapping)
    L.check_error(status, "infiniopCreatePagedCachingDescriptor")
    size = c_size_t(123)
    L.check_error(L.LIBINFINIOP.infiniopGetPagedCachingWorkspaceSize(op, ctypes.byref(size)))
    assert size.value == 0
    torch.cuda.synchronize()
    L.check_error(
        L.LIBINFINIOP.infiniopPagedCaching(op, c_void_p(0), 0, ptr(k_cache), ptr(v_cache), ptr(k), ptr(v),
                                           ptr(slot_mapping), c_void_p(stream or 0)),
        "infiniopPagedCaching",
    )
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedCachingDescriptor(op))
    return k_cache, v_cache


def create_rope_paged_caching(handle, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table, algo):
    descs = [describe(t) for t in (k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table)]
    op = L.infiniopOperatorDescriptor_t()
    status = L.LIBINFINIOP.infiniopCreateRoPEPagedCachingDescriptor(handle, ctypes.byref(op), *descs, int(algo))
    for d in descs:
        L.destroy_tensor_descriptor(d)
    return status, op


def run_rope_paged_caching(handle, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table, algo, stream=None):
    """In place on the device pools; returns them."""
    status, op = create_rope_paged_caching(handle, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table, algo)
    L.check_error(status, "infiniopCreateRoPEPagedCachingDescriptor")
    size = c_size_t(123)
    L.check_error(L.LIBINFINIOP.infiniopGetRoPEPagedCachingWorkspaceSize(op, ctypes.byref(size)))
    assert size.value == 0
    torch.cuda.synchronize()
    L.check_error(
        L.LIBINFINIOP.infiniopRoPEPagedCaching(op, c_void_p(0), 0, ptr(k_cache), ptr(v_cache), ptr(k), ptr(v),
                                               ptr(slot_mapping), ptr(pos_ids), ptr(sin_table), ptr(cos_table),
                                               c_void_p(stream or 0)),
        "infiniopRoPEPagedCaching",
    )
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(op))
    return k_cache, v_cache


def create_rope_qk_paged_caching(handle, q_out, q, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table, algo):
    descs = [describe(t) for t in (q_out, q, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table)]
    op = L.infiniopOperatorDescriptor_t()
    status = L.LIBINFINIOP.infiniopCreateRoPEQKPagedCachingDescriptor(handle, ctypes.byref(op), *descs, int(algo))
    for d in descs:
        L.destroy_tensor_descriptor(d)
    return status, op


def run_rope_qk_paged_caching(handle, q_out, q, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table, algo,
                              stream=None):
    """In place on the device pools and q_out; returns (k_cache, v_cache, q_out)."""
    status, op = create_rope_qk_paged_caching(handle, q_out, q, k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table,
                                              cos_table, algo)
    L.check_error(status, "infiniopCreateRoPEQKPagedCachingDescriptor")
    size = c_size_t(123)
    L.check_error(L.LIBINFINIOP.infiniopGetRoPEPagedCachingWorkspaceSize(op, ctypes.byref(size)))
    assert size.value == 0
    torch.cuda.synchronize()
    L.check_error(
        L.LIBINFINIOP.infiniopRoPEQKPagedCaching(op, c_void_p(0), 0, ptr(q_out), ptr(q), ptr(k_cache), ptr(v_cache), ptr(k),
                                                 ptr(v), ptr(slot_mapping), ptr(pos_ids), ptr(sin_table), ptr(cos_table),
                                                 c_void_p(stream or 0)),
        "infiniopRoPEQKPagedCaching",
    )
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(op))
    return k_cache, v_cache, q_out


def create_kv_caching(handle, k_cache, v_cache, k, v, past_kv_lengths):
    descs = [describe(t) for t in (k_cache, v_cache, k, v, past_kv_lengths)]
    op = L.infiniopOperatorDescriptor_t()
    status = L.LIBINFINIOP.infiniopCreateKVCachingDescriptor(handle, ctypes.byref(op), *descs)
    for d in descs:
        L.destroy_tensor_descriptor(d)
    return status, op


def run_kv_caching(handle, k_cache, v_cache, k, v, past_kv_lengths, stream=None):
    """In place on the device caches (the sequence of calls of test/infiniop/kv_caching.py:95-150); returns them."""
    status, op = create_kv_caching(handle, k_cache, v_cache, k, v, past_kv_lengths)
    L.check_error(status, "infiniopCreateKVCachingDescriptor")
    size = c_size_t(123)
    L.check_error(L.LIBINFINIOP.infiniopGetKVCachingWorkspaceSize(op, ctypes.byref(size)))
    assert size.value == 0
    torch.cuda.synchronize()
    L.check_error(
        L.LIBINFINIOP.infiniopKVCaching(op, c_void_p(0), 0, ptr(k_cache), ptr(v_cache), ptr(k), ptr(v),
                                        ptr(past_kv_lengths), c_void_p(stream or 0)),
        "infiniopKVCaching",
    )
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyKVCachingDescriptor(op))
    return k_cache, v_cache
