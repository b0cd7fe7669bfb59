"""The torch-facing operators of infinicore_amd.ops (argument order of the reference's Python ops)."""
import pytest
import torch

from infinicore_amd import workloads

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def test_paged_attention_and_caching_through_the_python_operators(oracle):
    from infinicore_amd import ops

    cfg = workloads.DecodeConfig("ops", torch.bfloat16, 4, 32, 8, 128, 16, 10, 1500, seed=77)
    inp = workloads.make_decode_inputs(cfg)
    q, k, v, bt, sl = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens)]
    want = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale).float()
    for _ in range(2):  # second call hits the plan cache
        got = ops.paged_attention(q, k, v, bt, sl, None, inp.scale)
        torch.cuda.synchronize()
        assert torch.all((got.float().cpu() - want).abs() <= 1e-2 + 2e-3 * want.abs())
    out = torch.empty_like(q)
    assert ops.paged_attention(q, k, v, bt, sl, scale=inp.scale, out=out) is out

    # one decode step: append one token per sequence with paged_caching, lengths grow by one
    new_k = torch.randn(4, 8, 128, device=DEV).to(torch.bfloat16)
    new_v = torch.randn(4, 8, 128, device=DEV).to(torch.bfloat16)
    slots = torch.stack([bt[s, int(sl[s]) // 16] * 16 + int(sl[s]) % 16 for s in range(4)])
    room = torch.tensor([int(sl[s]) // 16 < ((int(sl[s]) + 15) // 16) for s in range(4)])
    slots = torch.where(room.to(DEV), slots, torch.full_like(slots, -1))  # no free row in the last page: skip
    k_ret, v_ret = ops.paged_caching(k, v, new_k, new_v, slots)
    assert k_ret is k and v_ret is v
    k_want, v_want = oracle.paged_caching(inp.k_cache.clone(), inp.v_cache.clone(), new_k.cpu(), new_v.cpu(), slots.cpu())
    torch.cuda.synchronize()
    assert torch.equal(k.cpu().view(torch.int16), k_want.view(torch.int16))
    assert torch.equal(v.cpu().view(torch.int16), v_want.view(torch.int16))
    ops.clear_plan_cache()


def test_operators_refuse_host_tensors():
    from infinicore_amd import ops

    t = torch.zeros(1, 1, 128, dtype=torch.float16)
    with pytest.raises(ValueError):
        ops.paged_attention(t, t, t, t, t)
