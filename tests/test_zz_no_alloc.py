"""infiniopPagedAttentionNoAlloc (the call without a workspace argument: partial results in the library's own
per-device scratch array) against infiniopPagedAttention, through the C ABI: bit-identical outputs, on two
calls in a row of which the second is the smaller, each also within atol 1e-2 / rtol 2e-3 of the CPU oracle's
unrounded result, and a clear refusal above the array's size."""
import ctypes
from ctypes import c_void_p

import pytest
import torch

from infinicore_amd import libinfiniop as L
from infinicore_amd import workloads
from tests import capi

pytestmark = pytest.mark.gpu


def _both_ways(handle, cfg, oracle):
    dev = torch.device("cuda:0")
    inp = workloads.make_decode_inputs(cfg)
    q, kc, vc, bt, sl = (t.to(dev) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens))
    want = capi.run_paged_attention(handle, q, kc, vc, bt, sl, inp.scale)
    got = torch.zeros_like(want)
    status, op = capi.create_paged_attention(handle, got, q, kc, vc, bt, sl, None, inp.scale)
    L.check_error(status)
    size = capi.workspace_size_attention(op)
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopPagedAttentionNoAlloc(op, capi.ptr(got), capi.ptr(q), capi.ptr(kc), capi.ptr(vc),
                                                              capi.ptr(bt), capi.ptr(sl), c_void_p(0), c_void_p(0)),
                  "infiniopPagedAttentionNoAlloc")
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))
    # the entry point against the oracle itself, not only against its sibling
    _, exact = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                      num_threads=8, return_fp32=True)
    err = (got.float().cpu() - exact).abs()
    assert torch.all(err <= 1e-2 + 2e-3 * exact.abs()), f"{cfg.name}: max abs err {err.max().item():.4g} against the oracle"
    return want, got, size


def test_two_calls_in_a_row_the_second_smaller(gpu_handle, oracle):
    # both use partial results (sequences cut across wavefronts), so both go through the scratch array
    big = workloads.DecodeConfig("noalloc_big", torch.bfloat16, 24, 32, 8, 128, 16, 300, 3000, seed=501)
    small = workloads.DecodeConfig("noalloc_small", torch.float16, 3, 16, 4, 128, 16, 100, 900, seed=502)
    for cfg in (big, small):
        want, got, size = _both_ways(gpu_handle, cfg, oracle)
        assert size > 0, "the case must need scratch to test anything"
        assert torch.equal(want.view(torch.int16), got.view(torch.int16)), cfg.name


def test_latent_attention_goes_through_the_array_too(gpu_handle, oracle):
    cfg = workloads.DecodeConfig("noalloc_mla", torch.bfloat16, 4, 16, 1, 576, 16, 200, 1200, seed=503, value_size=512)
    want, got, size = _both_ways(gpu_handle, cfg, oracle)
    assert size > 0
    assert torch.equal(want.view(torch.int16), got.view(torch.int16))


def test_refuses_a_descriptor_that_needs_more_than_the_array(gpu_handle, capfd):
    """128 sequences x 128 latent heads on fixed partitions need far more than 32 MiB of partial results."""
    dev = torch.device("cuda:0")
    q = torch.zeros((300, 128, 576), dtype=torch.bfloat16, device=dev)
    out = torch.zeros((300, 128, 512), dtype=torch.bfloat16, device=dev)
    kc = torch.zeros((8, 1, 16, 576), dtype=torch.bfloat16, device=dev)
    vc = torch.zeros((8, 1, 16, 512), dtype=torch.bfloat16, device=dev)
    bt = torch.zeros((300, 512), dtype=torch.int64, device=dev)
    sl = torch.zeros((300,), dtype=torch.int64, device=dev)
    status, op = capi.create_paged_attention(gpu_handle, out, q, kc, vc, bt, sl, None, 0.1)
    L.check_error(status)
    assert capi.workspace_size_attention(op) > (32 << 20)
    status = L.LIBINFINIOP.infiniopPagedAttentionNoAlloc(op, capi.ptr(out), capi.ptr(q), capi.ptr(kc), capi.ptr(vc),
                                                         capi.ptr(bt), capi.ptr(sl), c_void_p(0), c_void_p(0))
    assert status == L.InfiniStatus.INSUFFICIENT_WORKSPACE
    assert "infiniopPagedAttentionNoAlloc" in capfd.readouterr().err
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))
