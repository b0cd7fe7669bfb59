"""GPU parity of infiniopPagedCaching (through the C ABI): bit-exact against the CPU oracle."""
import pytest
import torch

from infinicore_amd import workloads

from capi import run_paged_caching

pytestmark = pytest.mark.gpu


def bits(t):
    return t.contiguous().view(torch.int16 if t.element_size() == 2 else torch.int32)


def test_c5_prefill_scatter_bit_exact(gpu_handle, oracle):
    inp = workloads.make_caching_inputs(workloads.CACHING_CONFIGS["c5_prefill_scatter"])
    dev = torch.device("cuda:0")
    k_cache, v_cache = inp.k_cache.to(dev), inp.v_cache.to(dev)
    print("case c5 tokens", inp.k.shape[0], "padding", int((inp.slot_mapping < 0).sum()), flush=True)
    run_paged_caching(gpu_handle, k_cache, v_cache, inp.k.to(dev), inp.v.to(dev), inp.slot_mapping.to(dev))
    k_want, v_want = oracle.paged_caching(inp.k_cache.clone(), inp.v_cache.clone(), inp.k, inp.v, inp.slot_mapping)
    assert torch.equal(bits(k_cache.cpu()), bits(k_want))
    assert torch.equal(bits(v_cache.cpu()), bits(v_want))
