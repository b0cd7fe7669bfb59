"""GPU parity of infiniopPagedAttention (through the C ABI) against the CPU oracle.

Tolerance is the one the task fixes for fp16 / bf16 attention output: atol 1e-2, rtol 2e-3
(torch.allclose semantics: |got - want| <= atol + rtol * |want|).
"""
import os

import numpy as np
import pytest
import torch

from infinicore_amd import workloads

from capi import run_paged_attention

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 2e-3
ORACLE_THREADS = min(16, os.cpu_count() or 1)


def assert_close(got, want, what=""):
    got, want = got.float().cpu(), want.float().cpu()
    err = (got - want).abs()
    bound = ATOL + RTOL * want.abs()
    worst = (err - bound).max().item()
    assert worst <= 0, f"{what}: max abs err {err.max().item():.4g}, exceeds atol/rtol bound by {worst:.4g}"


def to_device(inp):
    dev = torch.device("cuda:0")
    return [t.to(dev) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens)]


def run_case(gpu_handle, oracle, inp, alibi=None, num_threads=ORACLE_THREADS):
    q, k, v, bt, sl = to_device(inp)
    alibi_dev = alibi.to(q.device) if alibi is not None else None
    print(f"case {inp.config.name} B={q.shape[0]} H={q.shape[1]} Hkv={k.shape[1]} D={q.shape[2]} "
          f"bs={k.shape[2]} dtype={q.dtype} lens[:4]={inp.seq_lens[:4].tolist()}", flush=True)
    got = run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale, alibi=alibi_dev)
    want = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                  alibi_slopes=alibi, num_threads=num_threads)
    assert_close(got, want, inp.config.name)
    return got, want


def custom(name, dtype, B, H, Hkv, D, bs, lo, hi, seed, **kw):
    return workloads.DecodeConfig(name, dtype, B, H, Hkv, D, bs, lo, hi, seed=seed, **kw)


def test_c1_plumbing_mha(gpu_handle, oracle):
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c1_plumbing_mha"]))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(
    "B,H,Hkv,D,bs,max_len",
    [
        # the reference's own test list, test/infiniop/paged_attention.py:95-101 (head sizes 64 / 128)
        (1, 1, 1, 128, 16, 1024),
        (4, 40, 40, 128, 16, 1024),
        (6, 40, 40, 128, 16, 1024),
        (3, 8, 8, 128, 16, 1024),
        (3, 8, 8, 64, 16, 1024),
        (8, 64, 8, 128, 16, 2048),
    ],
)
def test_reference_test_shapes(gpu_handle, oracle, dtype, B, H, Hkv, D, bs, max_len):
    cfg = custom(f"ref_{B}_{H}_{Hkv}_{D}", dtype, B, H, Hkv, D, bs, 1, max_len - 1, seed=7 * B + H + D)
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(cfg))


def test_c2_llama3_8b_full_size(gpu_handle, oracle):
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c2_llama3_8b_b32"]))


def test_c2_generic_kernel_matches(gpu_handle, oracle, monkeypatch):
    """The element-wise fallback kernel is a second device implementation; on a reduced c2 it must
    agree with the oracle as well."""
    monkeypatch.setenv("INFINIOP_AMD_PA_KERNEL", "generic")
    cfg = custom("c2_small_generic", torch.bfloat16, 4, 32, 8, 128, 16, 512, 2048, seed=5)
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(cfg))
