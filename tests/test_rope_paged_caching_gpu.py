"""GPU parity of infiniopRoPEPagedCaching (through the C ABI) against the CPU oracle: bit-exact pool contents."""
import ctypes

import pytest
import torch

from infinicore_amd import libinfiniop as L

from capi import create_rope_paged_caching, ptr, run_paged_caching, run_rope_paged_caching
from test_rope_paged_caching_cpu import tables

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
J, NEOX = L.RoPEAlgo.GPT_J, L.RoPEAlgo.GPT_NEOX


def bits(t):
    return t.cpu().view(torch.int32 if t.dtype == torch.float32 else torch.int16)


def make(dtype, ntok, H, D, Dv=None, bs=16, NB=None, table_len=4096, seed=0, pad_every=9):
    Dv = Dv or D
    NB = NB or (ntok + bs - 1) // bs + 3
    g = torch.Generator().manual_seed(seed)
    k = torch.randn((ntok, H, D), generator=g).to(dtype)
    v = torch.randn((ntok, H, Dv), generator=g).to(dtype)
    slots = torch.randperm(NB * bs, generator=g)[:ntok].to(torch.int64)
    if pad_every:
        slots[::pad_every] = -1
    pos = torch.randint(0, table_len, (ntok,), generator=g)
    sin, cos = tables(table_len, D, dtype)
    k_cache = torch.full((NB, H, bs, D), 7.0, dtype=dtype)
    v_cache = torch.full((NB, H, bs, Dv), -3.0, dtype=dtype)
    return [k_cache, v_cache, k, v, slots, pos, sin, cos]


def check(gpu_handle, oracle, case, algo, what=""):
    print(f"case {what} k {tuple(case[2].shape)} {case[2].dtype} algo {algo}", flush=True)
    dev = [t.to(DEV) for t in case]
    run_rope_paged_caching(gpu_handle, *dev, algo)
    want_k, want_v = case[0].clone(), case[1].clone()
    oracle.rope_paged_caching(want_k, want_v, *case[2:], algo == NEOX)
    assert torch.equal(bits(dev[0]), bits(want_k)), f"{what}: K pool differs"
    assert torch.equal(bits(dev[1]), bits(want_v)), f"{what}: V pool differs"
    return dev


@pytest.mark.parametrize("algo", [J, NEOX], ids=["gpt_j", "gpt_neox"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_decode_step_one_token_per_sequence(gpu_handle, oracle, dtype, algo):
    """The Llama-3-8B batch-32 decode step: 32 tokens x 8 KV heads x 128."""
    check(gpu_handle, oracle, make(dtype, 32, 8, 128, seed=1, pad_every=0), algo, "decode step")


@pytest.mark.parametrize("algo", [J, NEOX], ids=["gpt_j", "gpt_neox"])
def test_prefill_chunk_with_padding(gpu_handle, oracle, algo):
    """4096 tokens x 8 x 128 bf16 into a 65536-slot pool, every ninth entry padding."""
    check(gpu_handle, oracle, make(torch.bfloat16, 4096, 8, 128, NB=4096, seed=2), algo, "prefill chunk")


@pytest.mark.parametrize("algo", [J, NEOX], ids=["gpt_j", "gpt_neox"])
@pytest.mark.parametrize("H,D,Dv", [(8, 64, 64), (4, 192, 192), (2, 256, 256), (1, 576, 512), (3, 32, 80), (40, 128, 128)])
def test_head_sizes_and_counts(gpu_handle, oracle, H, D, Dv, algo):
    """Heads of 64 / 192 / 256, the latent-attention pair 576 / 512, values wider than keys, 40 heads (more than a
    workgroup's box holds in one step)."""
    check(gpu_handle, oracle, make(torch.float16, 50, H, D, Dv, seed=D + H), algo, f"H{H} D{D}")


@pytest.mark.parametrize("algo", [J, NEOX], ids=["gpt_j", "gpt_neox"])
@pytest.mark.parametrize("D,Dv", [(36, 36), (20, 24), (128, 100)])
def test_sizes_that_are_not_multiples_of_16_bytes(gpu_handle, oracle, D, Dv, algo):
    """Half-vectors of 18 and 10 elements and a value row of 200 bytes: one pair / one element per step."""
    check(gpu_handle, oracle, make(torch.bfloat16, 21, 3, D, Dv, seed=D), algo, f"odd D{D}")


@pytest.mark.parametrize("pos_dtype", [torch.int32, torch.uint8, torch.int16, torch.uint16, torch.uint32, torch.uint64, torch.int8])
def test_position_dtypes(gpu_handle, oracle, pos_dtype):
    case = make(torch.float16, 40, 4, 64, table_len=100, seed=31)
    case[5] = case[5].to(pos_dtype)
    check(gpu_handle, oracle, case, NEOX, f"pos {pos_dtype}")


def test_positions_outside_the_tables_and_slots_outside_the_pool(gpu_handle, oracle):
    """Positions below 0 / beyond the last row use the nearest row; slots beyond the pool are dropped like padding."""
    case = make(torch.bfloat16, 16, 2, 64, table_len=50, NB=2, seed=37, pad_every=0)
    case[5] = torch.tensor([0, 49, 50, 10 ** 9, -1, -10 ** 6, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12])
    case[4][3], case[4][8] = 2 * 16, 10 ** 12  # first slot past the pool, and far past it
    dev = [t.to(DEV) for t in case]
    run_rope_paged_caching(gpu_handle, *dev, J)
    want_k, want_v = case[0].clone(), case[1].clone()
    inside = case[4].clone()
    inside[3], inside[8] = -1, -1
    oracle.rope_paged_caching(want_k, want_v, case[2], case[3], inside, case[5], case[6], case[7], False)
    assert torch.equal(bits(dev[0]), bits(want_k)) and torch.equal(bits(dev[1]), bits(want_v))


@pytest.mark.parametrize("algo", [J, NEOX], ids=["gpt_j", "gpt_neox"])
def test_permuted_pool_layout_strided_sources_and_unaligned_bases(gpu_handle, oracle, algo):
    """Pools stored [pages, rows, heads, d] and handed over permuted (test/infinicore/ops/paged_caching.py:22-34),
    k and v as every other token of a longer tensor; then every operand shifted by one element."""
    case = make(torch.float16, 24, 4, 64, seed=41)
    kc, vc, k, v = case[:4]
    kc_dev = kc.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)
    vc_dev = vc.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)
    k_wide = torch.zeros((48, 4, 64), dtype=k.dtype, device=DEV)
    v_wide = torch.zeros((48, 4, 64), dtype=v.dtype, device=DEV)
    k_wide[::2], v_wide[::2] = k.to(DEV), v.to(DEV)
    rest = [t.to(DEV) for t in case[4:]]
    run_rope_paged_caching(gpu_handle, kc_dev, vc_dev, k_wide[::2], v_wide[::2], *rest, algo)
    want_k, want_v = kc.clone(), vc.clone()
    oracle.rope_paged_caching(want_k, want_v, *case[2:], algo == NEOX)
    assert torch.equal(bits(kc_dev.contiguous()), bits(want_k)) and torch.equal(bits(vc_dev.contiguous()), bits(want_v))

    def shifted(t):
        flat = torch.zeros(t.numel() + 1, dtype=t.dtype, device=DEV)
        view = flat[1:].view(t.shape)
        view.copy_(t)
        return view

    dev = [shifted(t) if i in (0, 1, 2, 3, 6, 7) else t.to(DEV) for i, t in enumerate(case)]
    run_rope_paged_caching(gpu_handle, *dev, algo)
    assert torch.equal(bits(dev[0]), bits(want_k)) and torch.equal(bits(dev[1]), bits(want_v))


def test_identity_rotation_leaves_what_paged_caching_leaves(gpu_handle):
    """Device against device: sin = 0, cos = 1 must give the pools infiniopPagedCaching gives."""
    case = make(torch.bfloat16, 300, 8, 128, seed=43)
    case[6], case[7] = torch.zeros_like(case[6]), torch.ones_like(case[7])
    fused = [t.to(DEV) for t in case]
    plain = [t.to(DEV) for t in case[:5]]
    run_rope_paged_caching(gpu_handle, *fused, NEOX)
    run_paged_caching(gpu_handle, *plain)
    assert torch.equal(fused[0], plain[0]) and torch.equal(fused[1], plain[1])


def test_capture_and_replay(gpu_handle, oracle):
    """One launch, no allocation, no synchronisation: recordable; replays after the inputs changed follow them."""
    case = make(torch.float16, 32, 8, 128, seed=47, pad_every=0)
    dev = [t.to(DEV) for t in case]
    status, op = create_rope_paged_caching(gpu_handle, *dev, NEOX)
    assert status == 0
    rt = L.LIBINFINIRT
    stream, graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    L.check_error(rt.infinirtStreamCreate(ctypes.byref(stream)))
    torch.cuda.synchronize()

    def call():
        L.check_error(L.LIBINFINIOP.infiniopRoPEPagedCaching(op, None, 0, *[ptr(t) for t in dev], stream))

    L.check_error(rt.infinirtStreamBeginCapture(stream, 0))
    call()
    L.check_error(rt.infinirtStreamEndCapture(stream, ctypes.byref(graph)))
    L.check_error(rt.infinirtGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0))
    for replay in range(3):
        new_pos = (case[5] + 17 * replay) % 4096
        dev[5].copy_(new_pos)
        dev[0].fill_(7.0)
        torch.cuda.synchronize()
        L.check_error(rt.infinirtGraphLuanch(graph_exec, stream))
        L.check_error(rt.infinirtStreamSynchronize(stream))
        want_k, want_v = case[0].clone(), case[1].clone()
        oracle.rope_paged_caching(want_k, want_v, case[2], case[3], case[4], new_pos, case[6], case[7], True)
        assert torch.equal(bits(dev[0]), bits(want_k)), f"replay {replay}"
    L.check_error(rt.infinirtGraphExecDestroy(graph_exec))
    L.check_error(rt.infinirtGraphDestroy(graph))
    L.check_error(rt.infinirtStreamDestroy(stream))
    L.check_error(L.LIBINFINIOP.infiniopDestroyRoPEPagedCachingDescriptor(op))


def test_python_operator_then_attention_sees_the_rotated_keys(gpu_handle, oracle):
    """Through infinicore_amd.ops: rotate-and-scatter a decode step's K / V, then attend over the pool; the
    attention output must be that of the oracle on the oracle's pools."""
    from infinicore_amd import ops

    torch.manual_seed(5)
    B, H, Hkv, D, bs, L0 = 4, 16, 4, 128, 16, 37
    nb = B * 4
    k_pool = torch.randn((nb, Hkv, bs, D)).to(torch.bfloat16)
    v_pool = torch.randn((nb, Hkv, bs, D)).to(torch.bfloat16)
    bt = torch.arange(nb, dtype=torch.int64).view(B, 4)
    lens = torch.full((B,), L0 + 1, dtype=torch.int64)
    k_new, v_new = torch.randn((B, Hkv, D)).to(torch.bfloat16), torch.randn((B, Hkv, D)).to(torch.bfloat16)
    slots = bt[:, L0 // bs] * bs + L0 % bs
    pos = torch.full((B,), L0, dtype=torch.int64)
    sin, cos = tables(128, D, torch.bfloat16)
    q = torch.randn((B, H, D)).to(torch.bfloat16)
    kd, vd = k_pool.to(DEV), v_pool.to(DEV)
    ops.rope_paged_caching(kd, vd, k_new.to(DEV), v_new.to(DEV), slots.to(DEV), pos.to(DEV), sin.to(DEV), cos.to(DEV),
                           L.RoPEAlgo.GPT_NEOX)
    out = ops.paged_attention(q.to(DEV), kd, vd, bt.to(DEV), lens.to(DEV), None, D ** -0.5)
    torch.cuda.synchronize()
    oracle.rope_paged_caching(k_pool, v_pool, k_new, v_new, slots, pos, sin, cos, True)
    assert torch.equal(bits(kd), bits(k_pool))
    _, want = oracle.paged_attention(q, k_pool, v_pool, bt, lens, D ** -0.5, return_fp32=True)
    err = (out.float().cpu() - want).abs()
    assert bool((err <= 1e-2 + 2e-3 * want.abs()).all()), err.max()


# ---- the query rotated in the same launch (infiniopRoPEQKPagedCaching) ------------------------------------------

def check_qk(gpu_handle, oracle, case, q, algo, what="", q_out=None, in_place=False):
    """Pools against the fused oracle function, q_out against the rotation on its own (every token, padding too)."""
    from capi import run_rope_qk_paged_caching

    print(f"case {what} q {tuple(q.shape)} k {tuple(case[2].shape)} {q.dtype} algo {algo} in_place {in_place}", flush=True)
    dev = [t.to(DEV) for t in case]
    q_dev = q.to(DEV)
    out_dev = q_dev if in_place else (q_out.to(DEV) if q_out is not None else torch.full(q.shape, 5.0, dtype=q.dtype, device=DEV))
    run_rope_qk_paged_caching(gpu_handle, out_dev, q_dev, *dev, algo)
    want_k, want_v = case[0].clone(), case[1].clone()
    oracle.rope_paged_caching(want_k, want_v, *case[2:], algo == NEOX)
    want_q = oracle.rope(q, case[5], case[6], case[7], algo == NEOX)
    assert torch.equal(bits(dev[0]), bits(want_k)), f"{what}: K pool differs"
    assert torch.equal(bits(dev[1]), bits(want_v)), f"{what}: V pool differs"
    assert torch.equal(bits(out_dev.contiguous()), bits(want_q)), f"{what}: rotated query differs"
    if not in_place:
        assert torch.equal(bits(q_dev), bits(q)), f"{what}: the query operand was written"
    return dev, out_dev


@pytest.mark.parametrize("algo", [J, NEOX], ids=["gpt_j", "gpt_neox"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_query_decode_step(gpu_handle, oracle, dtype, algo):
    """The Llama-3-8B batch-32 decode step with its 32 query heads."""
    case = make(dtype, 32, 8, 128, seed=51, pad_every=0)
    q = torch.randn((32, 32, 128), generator=torch.Generator().manual_seed(52)).to(dtype)
    check_qk(gpu_handle, oracle, case, q, algo, "decode step with query")


@pytest.mark.parametrize("in_place", [False, True])
@pytest.mark.parametrize("algo", [J, NEOX], ids=["gpt_j", "gpt_neox"])
def test_query_prefill_chunk_padding_tokens_are_rotated_too(gpu_handle, oracle, algo, in_place):
    case = make(torch.bfloat16, 1000, 8, 128, NB=1200, seed=53)  # every ninth slot is padding
    q = torch.randn((1000, 32, 128), generator=torch.Generator().manual_seed(54)).to(torch.bfloat16)
    check_qk(gpu_handle, oracle, case, q, algo, "prefill chunk with query", in_place=in_place)


@pytest.mark.parametrize("Hq,Hkv,D,Dv", [(1, 1, 64, 64), (5, 5, 64, 128), (48, 3, 256, 64), (16, 1, 576, 512), (7, 2, 24, 40)])
def test_query_head_counts_and_sizes(gpu_handle, oracle, Hq, Hkv, D, Dv):
    case = make(torch.float16, 77, Hkv, D, Dv=Dv, seed=55 + Hq)
    q = torch.randn((77, Hq, D), generator=torch.Generator().manual_seed(56)).to(torch.float16)
    check_qk(gpu_handle, oracle, case, q, NEOX if Hq % 2 else J, f"Hq={Hq} Hkv={Hkv} D={D}/{Dv}")


def test_query_key_and_value_as_slices_of_one_projection_output(gpu_handle, oracle):
    """q, k, v are column slices of one [tokens, (Hq + 2 Hkv) D] tensor, rotated in place / scattered from there."""
    from capi import run_rope_qk_paged_caching

    ntok, Hq, Hkv, D = 200, 16, 4, 128
    case = make(torch.bfloat16, ntok, Hkv, D, seed=61)
    g = torch.Generator().manual_seed(62)
    fused = torch.randn((ntok, (Hq + 2 * Hkv) * D), generator=g).to(torch.bfloat16)
    fused[:, Hq * D:(Hq + Hkv) * D] = case[2].reshape(ntok, -1)
    fused[:, (Hq + Hkv) * D:] = case[3].reshape(ntok, -1)
    fused_dev = fused.to(DEV)
    q_dev = fused_dev[:, :Hq * D].view(ntok, Hq, D)
    k_dev = fused_dev[:, Hq * D:(Hq + Hkv) * D].view(ntok, Hkv, D)
    v_dev = fused_dev[:, (Hq + Hkv) * D:].view(ntok, Hkv, D)
    assert not q_dev.is_contiguous() and not k_dev.is_contiguous()
    dev = [t.to(DEV) for t in case]
    run_rope_qk_paged_caching(gpu_handle, q_dev, q_dev, dev[0], dev[1], k_dev, v_dev, *dev[4:], NEOX)
    want_k, want_v = case[0].clone(), case[1].clone()
    oracle.rope_paged_caching(want_k, want_v, *case[2:], True)
    want_q = oracle.rope(fused[:, :Hq * D].reshape(ntok, Hq, D), case[5], case[6], case[7], True)
    assert torch.equal(bits(dev[0]), bits(want_k)) and torch.equal(bits(dev[1]), bits(want_v))
    assert torch.equal(bits(q_dev.contiguous()), bits(want_q))
    assert torch.equal(bits(fused_dev[:, Hq * D:].contiguous()), bits(fused[:, Hq * D:].contiguous())), "k / v columns were written"


def test_query_unaligned_and_padded_operands_take_the_pair_at_a_time_path(gpu_handle, oracle):
    from capi import run_rope_qk_paged_caching

    case = make(torch.float16, 50, 3, 64, seed=63)
    q = torch.randn((50, 6, 64), generator=torch.Generator().manual_seed(64)).to(torch.float16)
    dev = [t.to(DEV) for t in case]
    raw = torch.zeros(q.numel() + 1, dtype=q.dtype, device=DEV)
    q_dev = raw[1:].view(q.shape)  # 2 bytes off a 16-byte boundary
    q_dev.copy_(q)
    out_dev = torch.full((50, 6, 72), 5.0, dtype=q.dtype, device=DEV)[:, :, :64]  # padded heads
    run_rope_qk_paged_caching(gpu_handle, out_dev, q_dev, *dev, J)
    want_k, want_v = case[0].clone(), case[1].clone()
    oracle.rope_paged_caching(want_k, want_v, *case[2:], False)
    assert torch.equal(bits(dev[0]), bits(want_k)) and torch.equal(bits(dev[1]), bits(want_v))
    assert torch.equal(bits(out_dev.contiguous()), bits(oracle.rope(q, case[5], case[6], case[7], False)))


def test_query_python_operator(gpu_handle, oracle):
    from infinicore_amd import ops

    case = make(torch.bfloat16, 32, 8, 128, seed=65, pad_every=0)
    q = torch.randn((32, 32, 128), generator=torch.Generator().manual_seed(66)).to(torch.bfloat16)
    dev = [t.to(DEV) for t in case]
    q_dev = q.to(DEV)
    kd, vd, qd = ops.rope_paged_caching(*dev, L.RoPEAlgo.GPT_NEOX, q=q_dev)
    torch.cuda.synchronize()
    assert qd is q_dev
    want_k, want_v = case[0].clone(), case[1].clone()
    oracle.rope_paged_caching(want_k, want_v, *case[2:], True)
    assert torch.equal(bits(kd), bits(want_k)) and torch.equal(bits(vd), bits(want_v))
    assert torch.equal(bits(qd), bits(oracle.rope(q, case[5], case[6], case[7], True)))
