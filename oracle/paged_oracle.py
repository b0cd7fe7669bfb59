"""Python front of the CPU oracle (test infrastructure only - see the header of paged_oracle.c).

Two independent restatements of the reference live here:

* the C oracle ``liboracle.so`` (device-kernel arithmetic: fp32 online softmax in the log2 domain,
  ``1 / (l + 1e-6)``, round-to-nearest-even), reached through ctypes on torch CPU tensors;
* ``torch_reference_attention`` / ``torch_reference_prefill`` / ``torch_reference_caching``: the torch functions the reference's
  own tests compare against (``test/infiniop/paged_attention.py:38-88``: gather the sequence's
  tokens through the block table, repeat KV heads for GQA, logits = scale * einsum in the storage
  dtype, softmax in fp32, probabilities cast back to the storage dtype, einsum with V;
  ``test/infiniop/paged_caching.py:25-55``: per-token assignment into a clone of the pools).
  ``vectorised=True`` computes the same thing without the per-token Python loop.
"""
from __future__ import annotations

import ctypes
import subprocess
from ctypes import POINTER, Structure, c_float, c_int, c_int64, c_void_p
from pathlib import Path

import torch

_DIR = Path(__file__).resolve().parent
_LIB_PATH = _DIR / "lib" / "liboracle.so"
_lib = None

DTYPE_CODE = {torch.float16: 0, torch.bfloat16: 1}


class AttentionShape(Structure):
    _fields_ = [("dtype", c_int)] + [
        (name, c_int64)
        for name in (
            "num_seqs", "num_heads", "num_kv_heads", "head_size", "value_size", "block_size", "max_blocks_per_seq",
            "q_stride", "q_head_stride", "o_stride", "o_head_stride",
            "k_batch_stride", "k_head_stride", "k_row_stride",
            "v_batch_stride", "v_head_stride", "v_row_stride",
            "block_table_stride",
        )
    ] + [("scale", c_float)]


class CachingShape(Structure):
    _fields_ = [
        (name, c_int64)
        for name in (
            "elem_size", "num_tokens", "num_kv_heads", "head_size", "v_head_size", "block_size",
            "k_src_stride", "v_src_stride", "k_cache_block_stride", "v_cache_block_stride",
            "k_cache_head_stride", "v_cache_head_stride", "k_cache_slot_stride", "v_cache_slot_stride",
        )
    ]


class KVCachingShape(Structure):
    _fields_ = [(name, c_int64) for name in ("elem_size", "batch_size", "num_kv_heads", "max_seq_len", "seq_len",
                                             "hidden_dim")] + [
        (name, c_int64 * 4) for name in ("k_cache_strides", "v_cache_strides", "k_strides", "v_strides")]


def build() -> None:
    proc = subprocess.run(["make", "-C", str(_DIR)], capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building the CPU oracle failed:\n" + proc.stdout + proc.stderr)


def load():
    global _lib
    if _lib is None:
        if not _LIB_PATH.is_file():
            build()
        lib = ctypes.CDLL(str(_LIB_PATH))
        common = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(AttentionShape)]
        lib.oracle_paged_attention.argtypes = [c_void_p] + common + [c_int]
        lib.oracle_paged_attention.restype = c_int
        lib.oracle_paged_attention_splitkv.argtypes = common + [c_int, c_int]
        lib.oracle_paged_attention_splitkv.restype = c_int
        lib.oracle_paged_attention_prefill.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                       c_void_p, c_void_p, POINTER(AttentionShape), c_int64, c_void_p,
                                                       c_int64, c_int]
        lib.oracle_paged_attention_prefill.restype = c_int
        lib.oracle_paged_caching.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(CachingShape)]
        lib.oracle_paged_caching.restype = c_int
        lib.oracle_rope_paged_caching.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                  c_void_p, c_int64, c_int, c_int, POINTER(CachingShape)]
        lib.oracle_rope_paged_caching.restype = c_int
        lib.oracle_rope.argtypes = [c_void_p] * 5 + [c_int64, c_int, c_int] + [c_int64] * 7
        lib.oracle_rope.restype = c_int
        lib.oracle_kv_caching.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, POINTER(KVCachingShape)]
        lib.oracle_kv_caching.restype = c_int
        lib.oracle_to_float.argtypes = [ctypes.c_uint16, c_int]
        lib.oracle_to_float.restype = c_float
        lib.oracle_from_float.argtypes = [c_float, c_int]
        lib.oracle_from_float.restype = ctypes.c_uint16
        _lib = lib
    return _lib


def _cpu(t: torch.Tensor) -> torch.Tensor:
    if t.is_cuda:
        raise ValueError("the oracle works on host tensors")
    return t


def paged_attention(q, k_cache, v_cache, block_tables, seq_lens, scale, alibi_slopes=None, *, out=None,
                    num_splits: int | None = None, num_threads: int = 1, return_fp32: bool = False):
    """C oracle on torch CPU tensors (any strides with a packed last dimension). ``num_splits`` selects
    the split-KV + combine formulation instead of the single pass. ``return_fp32`` also returns the
    result as the kernel holds it before rounding to the storage dtype (rows of empty sequences NaN)."""
    lib = load()
    q, k_cache, v_cache = _cpu(q), _cpu(k_cache), _cpu(v_cache)
    block_tables = _cpu(block_tables).to(torch.int64).contiguous()
    seq_lens = _cpu(seq_lens).to(torch.int64).contiguous()
    if out is None:
        out = torch.zeros((*q.shape[:-1], v_cache.shape[-1]), dtype=q.dtype)
    assert q.stride(-1) == 1 and out.stride(-1) == 1 and k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
    s = AttentionShape(
        DTYPE_CODE[q.dtype], q.shape[0], q.shape[1], k_cache.shape[1], q.shape[2], v_cache.shape[3], k_cache.shape[2],
        block_tables.shape[1], q.stride(0), q.stride(1), out.stride(0), out.stride(1),
        k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
        v_cache.stride(0), v_cache.stride(1), v_cache.stride(2),
        block_tables.stride(0), float(scale),
    )
    alibi_ptr = None
    if alibi_slopes is not None:
        alibi_slopes = _cpu(alibi_slopes).to(torch.float32).contiguous()
        alibi_ptr = alibi_slopes.data_ptr()
    args = [q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), block_tables.data_ptr(),
            seq_lens.data_ptr(), alibi_ptr, ctypes.byref(s)]
    out_f32 = None
    if num_splits is None:
        if return_fp32:
            out_f32 = torch.full((q.shape[0], q.shape[1], v_cache.shape[-1]), float("nan"), dtype=torch.float32)
        rc = lib.oracle_paged_attention(out.data_ptr(), out_f32.data_ptr() if return_fp32 else None, *args, num_threads)
    else:
        assert not return_fp32
        rc = lib.oracle_paged_attention_splitkv(out.data_ptr(), *args, num_splits, num_threads)
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return (out, out_f32) if return_fp32 else out


def paged_attention_prefill(q, k_cache, v_cache, block_tables, seq_lens, cum_seq_lens_q, scale, alibi_slopes=None, *,
                            out=None, rows=None, num_threads: int = 1, return_fp32: bool = False):
    """C oracle of the prefill operator on torch CPU tensors. ``rows`` (optional 1-D sequence of query
    row numbers) restricts the evaluation to those rows; all other rows of the result keep the content
    of ``out`` (zeros when ``out`` is not given; NaN in the fp32 result)."""
    lib = load()
    q, k_cache, v_cache = _cpu(q), _cpu(k_cache), _cpu(v_cache)
    block_tables = _cpu(block_tables).to(torch.int64).contiguous()
    seq_lens = _cpu(seq_lens).to(torch.int64).contiguous()
    cum = _cpu(cum_seq_lens_q).to(torch.int64).contiguous()
    if out is None:
        out = torch.zeros((*q.shape[:-1], v_cache.shape[-1]), dtype=q.dtype)
    assert q.stride(-1) == 1 and out.stride(-1) == 1 and k_cache.stride(-1) == 1 and v_cache.stride(-1) == 1
    assert cum.shape[0] == seq_lens.shape[0] + 1
    s = AttentionShape(
        DTYPE_CODE[q.dtype], seq_lens.shape[0], q.shape[1], k_cache.shape[1], q.shape[2], v_cache.shape[3],
        k_cache.shape[2], block_tables.shape[1], q.stride(0), q.stride(1), out.stride(0), out.stride(1),
        k_cache.stride(0), k_cache.stride(1), k_cache.stride(2),
        v_cache.stride(0), v_cache.stride(1), v_cache.stride(2),
        block_tables.stride(0), float(scale),
    )
    alibi_ptr = None
    if alibi_slopes is not None:
        alibi_slopes = _cpu(alibi_slopes).to(torch.float32).contiguous()
        alibi_ptr = alibi_slopes.data_ptr()
    rows_t, rows_ptr, num_rows = None, None, 0
    if rows is not None:
        rows_t = torch.as_tensor(rows, dtype=torch.int64).contiguous()
        rows_ptr, num_rows = rows_t.data_ptr(), rows_t.numel()
    out_f32 = None
    if return_fp32:
        out_f32 = torch.full((q.shape[0], q.shape[1], v_cache.shape[-1]), float("nan"), dtype=torch.float32)
    rc = lib.oracle_paged_attention_prefill(
        out.data_ptr(), out_f32.data_ptr() if return_fp32 else None, q.data_ptr(), k_cache.data_ptr(),
        v_cache.data_ptr(), block_tables.data_ptr(), seq_lens.data_ptr(), cum.data_ptr(), alibi_ptr, ctypes.byref(s),
        q.shape[0], rows_ptr, num_rows, num_threads)
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return (out, out_f32) if return_fp32 else out


def paged_caching(k_cache, v_cache, k, v, slot_mapping):
    """C oracle scatter; writes into ``k_cache`` / ``v_cache`` in place and returns them."""
    lib = load()
    slot_mapping = _cpu(slot_mapping).to(torch.int64).contiguous()
    s = CachingShape(
        k.element_size(), slot_mapping.shape[0], k.shape[1], k.shape[2], v.shape[2], k_cache.shape[2],
        k.stride(0), v.stride(0), k_cache.stride(0), v_cache.stride(0),
        k_cache.stride(1), v_cache.stride(1), k_cache.stride(2), v_cache.stride(2),
    )
    rc = lib.oracle_paged_caching(_cpu(k_cache).data_ptr(), _cpu(v_cache).data_ptr(), _cpu(k).data_ptr(),
                                  _cpu(v).data_ptr(), slot_mapping.data_ptr(), ctypes.byref(s))
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return k_cache, v_cache


def rope_paged_caching(k_cache, v_cache, k, v, slot_mapping, pos_ids, sin_table, cos_table, neox: bool):
    """C oracle rotary embedding of K fused with the scatter of K and V; writes into the caches in place and
    returns them. ``neox``: pairs half a vector apart (GPT-NeoX), else neighbouring (GPT-J)."""
    lib = load()
    slot_mapping = _cpu(slot_mapping).to(torch.int64).contiguous()
    pos_ids = _cpu(pos_ids).to(torch.int64).contiguous()
    sin_table, cos_table = _cpu(sin_table).contiguous(), _cpu(cos_table).contiguous()
    code = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}[k.dtype]
    s = CachingShape(
        k.element_size(), slot_mapping.shape[0], k.shape[1], k.shape[2], v.shape[2], k_cache.shape[2],
        k.stride(0), v.stride(0), k_cache.stride(0), v_cache.stride(0),
        k_cache.stride(1), v_cache.stride(1), k_cache.stride(2), v_cache.stride(2),
    )
    rc = lib.oracle_rope_paged_caching(_cpu(k_cache).data_ptr(), _cpu(v_cache).data_ptr(), _cpu(k).data_ptr(),
                                       _cpu(v).data_ptr(), slot_mapping.data_ptr(), pos_ids.data_ptr(), sin_table.data_ptr(),
                                       cos_table.data_ptr(), sin_table.shape[0], code, int(bool(neox)), ctypes.byref(s))
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return k_cache, v_cache


def rope(x, pos_ids, sin_table, cos_table, neox: bool, out=None):
    """C oracle rotary embedding of ``x`` [tokens, heads, d] (any token / head strides, packed last dimension), one
    position per token; returns the rotated tensor (``out``, which may be ``x``, or a new packed tensor)."""
    lib = load()
    x = _cpu(x)
    if out is None:
        out = torch.empty(x.shape, dtype=x.dtype)
    pos_ids = _cpu(pos_ids).to(torch.int64).contiguous()
    sin_table, cos_table = _cpu(sin_table).contiguous(), _cpu(cos_table).contiguous()
    assert x.stride(-1) == 1 and out.stride(-1) == 1 and out.shape == x.shape
    code = {torch.float16: 0, torch.bfloat16: 1, torch.float32: 2}[x.dtype]
    rc = lib.oracle_rope(out.data_ptr(), x.data_ptr(), pos_ids.data_ptr(), sin_table.data_ptr(), cos_table.data_ptr(),
                         sin_table.shape[0], code, int(bool(neox)), x.shape[0], x.shape[1], x.shape[2],
                         x.stride(0), x.stride(1), out.stride(0), out.stride(1))
    if rc != 0:
        raise ValueError("oracle rejected the arguments")
    return out


def torch_reference_rope(x, pos_ids, sin_table, cos_table, neox: bool):
    """The expected-value function of the reference's RoPE test on the CPU (test/infiniop/rope.py:84-121), restated:
    operands widened to fp32, ``t1 * cos - t2 * sin`` and ``t1 * sin + t2 * cos`` as separate tensor operations, one
    cast back. ``x`` is [tokens, heads, d]; returns the rotated tensor."""
    sin = sin_table[pos_ids.long()].float().unsqueeze(1)
    cos = cos_table[pos_ids.long()].float().unsqueeze(1)
    out = torch.empty_like(x)
    if neox:
        half = x.shape[-1] // 2
        t1, t2 = x[..., :half].float(), x[..., half:].float()
        out[..., :half] = (t1 * cos - t2 * sin).to(x.dtype)
        out[..., half:] = (t1 * sin + t2 * cos).to(x.dtype)
    else:
        t1, t2 = x[..., 0::2].float(), x[..., 1::2].float()
        out[..., 0::2] = (t1 * cos - t2 * sin).to(x.dtype)
        out[..., 1::2] = (t1 * sin + t2 * cos).to(x.dtype)
    return out


def kv_caching(k_cache, v_cache, k, v, past_kv_lengths):
    """C oracle append to contiguous caches; writes into ``k_cache`` / ``v_cache`` in place and returns them.
    Raises if a new token would land outside the cache (an out-of-bounds write in the reference)."""
    lib = load()
    past = _cpu(past_kv_lengths).to(torch.int64).contiguous()
    s = KVCachingShape(k.element_size(), k_cache.shape[0], k_cache.shape[1], k_cache.shape[2], k.shape[2], k_cache.shape[3],
                       (c_int64 * 4)(*k_cache.stride()), (c_int64 * 4)(*v_cache.stride()),
                       (c_int64 * 4)(*k.stride()), (c_int64 * 4)(*v.stride()))
    rc = lib.oracle_kv_caching(_cpu(k_cache).data_ptr(), _cpu(v_cache).data_ptr(), _cpu(k).data_ptr(),
                               _cpu(v).data_ptr(), past.data_ptr(), ctypes.byref(s))
    if rc != 0:
        raise ValueError("oracle rejected the arguments" if rc == -1 else "a new token lands outside the cache")
    return k_cache, v_cache


def torch_reference_kv_caching(k_cache, v_cache, k, v, past_kv_lengths):
    """The expected-value function of the reference's test (test/infiniop/kv_caching.py:23-33), restated."""
    seq_len = k.shape[2]
    for b in range(k_cache.shape[0]):
        past = int(past_kv_lengths[b])
        k_cache[b, :, past:past + seq_len, :] = k[b]
        v_cache[b, :, past:past + seq_len, :] = v[b]
    return k_cache, v_cache


# ---------------------------------------------------------------------------------------------------
# torch statement of the operators, as the reference's tests define the expected result
# ---------------------------------------------------------------------------------------------------

def _attend_one(query, keys, values, scale, bias):
    """query [1, H, D], keys / values [L, H, D]; test/infiniop/paged_attention.py:38-45."""
    logits = scale * torch.einsum("qhd,khd->hqk", query, keys).float()
    if bias is not None:
        logits = logits + bias.float()
    probs = torch.softmax(logits, dim=-1).to(values.dtype)
    return torch.einsum("hqk,khd->qhd", probs, values)


def torch_reference_attention(q, k_cache, v_cache, block_tables, seq_lens, scale, alibi_slopes=None,
                              vectorised: bool = True):
    """test/infiniop/paged_attention.py:48-88. Sequences with length 0 are left as zeros here (the
    reference test never draws one)."""
    num_heads, num_kv_heads = q.shape[1], v_cache.shape[1]
    group = num_heads // num_kv_heads
    block_size = v_cache.shape[2]
    out = torch.zeros((*q.shape[:-1], v_cache.shape[3]), dtype=q.dtype, device=q.device)
    for s in range(q.shape[0]):
        length = int(seq_lens[s])
        if length <= 0:
            continue
        if vectorised:
            pos = torch.arange(length, device=q.device)
            pages = block_tables[s].to(torch.int64)[pos // block_size]
            keys = k_cache[pages, :, pos % block_size, :]
            values = v_cache[pages, :, pos % block_size, :]
        else:
            k_rows, v_rows = [], []
            for t in range(length):
                page = int(block_tables[s, t // block_size])
                k_rows.append(k_cache[page, :, t % block_size, :])
                v_rows.append(v_cache[page, :, t % block_size, :])
            keys, values = torch.stack(k_rows), torch.stack(v_rows)
        if group > 1:
            keys = torch.repeat_interleave(keys, group, dim=1)
            values = torch.repeat_interleave(values, group, dim=1)
        bias = None
        if alibi_slopes is not None:
            rel = (torch.arange(length, device=q.device).int() - length + 1).float()
            bias = alibi_slopes.view(-1, 1, 1) * rel.view(1, 1, -1)
        out[s] = _attend_one(q[s].unsqueeze(0), keys, values, scale, bias).view(num_heads, -1)
    return out


def torch_reference_prefill(q, k_cache, v_cache, block_tables, seq_lens, cum_seq_lens_q, scale):
    """test/infiniop/paged_attention_prefill.py:88-125: per sequence, gather all of its K/V tokens, logits =
    einsum in the storage dtype -> fp32 * scale, add a -inf mask above position cache_len + q_idx, softmax in
    fp32 cast to the storage dtype, einsum with V. KV heads are repeated for grouped-query shapes (the
    reference test only draws num_heads == num_kv_heads, or one shared KV head)."""
    block_size = k_cache.shape[2]
    group = q.shape[1] // k_cache.shape[1]
    out = torch.zeros((*q.shape[:-1], v_cache.shape[3]), dtype=q.dtype, device=q.device)
    for i in range(len(cum_seq_lens_q) - 1):
        q0, q1 = int(cum_seq_lens_q[i]), int(cum_seq_lens_q[i + 1])
        num_new, total_len = q1 - q0, int(seq_lens[i])
        cache_len = total_len - num_new
        if num_new <= 0 or total_len <= 0:
            continue
        pos = torch.arange(total_len, device=q.device)
        pages = block_tables[i].to(torch.int64)[pos // block_size]
        keys = k_cache[pages, :, pos % block_size, :]
        values = v_cache[pages, :, pos % block_size, :]
        if group > 1:
            keys = torch.repeat_interleave(keys, group, dim=1)
            values = torch.repeat_interleave(values, group, dim=1)
        scores = torch.einsum("qhd,khd->hqk", q[q0:q1], keys).float() * scale
        limit = cache_len + torch.arange(num_new, device=q.device).view(-1, 1)
        mask = torch.where(pos.view(1, -1) <= limit, 0.0, float("-inf"))
        probs = torch.softmax(scores + mask.unsqueeze(0), dim=-1).to(q.dtype)
        out[q0:q1] = torch.einsum("hqk,khd->qhd", probs, values)
    return out


def torch_reference_caching(k_cache, v_cache, k, v, slot_mapping):
    """test/infiniop/paged_caching.py:25-55 (works on clones), extended to skip negative slots the way
    the device kernel does (the reference's torch function is never fed one)."""
    block_size = k_cache.shape[2]
    k_ref, v_ref = k_cache.clone(), v_cache.clone()
    for i in range(k.shape[0]):
        slot = int(slot_mapping[i])
        if slot < 0:
            continue
        k_ref[slot // block_size, :, slot % block_size, :] = k[i]
        v_ref[slot // block_size, :, slot % block_size, :] = v[i]
    return k_ref, v_ref
