"""GPU parity of infiniopPagedAttention (through the C ABI) against the CPU oracle.

Tolerance is the one the task fixes for fp16 / bf16 attention output: atol 1e-2, rtol 2e-3
(torch.allclose semantics: |got - want| <= atol + rtol * |want|).
"""
import ctypes
import os

import numpy as np
import pytest
import torch

from infinicore_amd import libinfiniop as L
from infinicore_amd import workloads

from capi import create_paged_attention, ptr, run_paged_attention, workspace_size_attention
from exact import exact_paged_attention

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 2e-3
ORACLE_THREADS = min(16, os.cpu_count() or 1)
DEV = "cuda:0"


@pytest.fixture(autouse=True)
def balanced_schedule_unless_the_test_says_otherwise(monkeypatch):
    """Small jobs are routed to the fixed-partition schedule by default; most cases here are small but are
    meant to exercise the work-equalising kernels, so that schedule is forced (tests that set the variable
    themselves override this; test_default_schedule_choice removes it)."""
    monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", "balanced")


def ulp_of(dtype, x):
    """Spacing of the storage dtype at |x|."""
    bits = 10 if dtype == torch.float16 else 7
    return torch.exp2(torch.floor(torch.log2(x.abs().clamp_min(2.0 ** -14))) - bits)


def assert_close(got, want, what="", want_f32=None):
    """The stated tolerance, element by element.

    `want_f32` is the oracle's result BEFORE its final rounding to fp16 / bf16. When it is given it is
    the yardstick: a device result that is the correctly rounded value of something within the
    tolerance of it always passes. Two results that were both rounded to bf16 can sit one bf16 step
    apart although they agree to 1e-6 before rounding, and above |x| = 2.44 one bf16 step (2^-6) is
    already more than atol + rtol * |x| - so against the ROUNDED oracle the check allows exactly that:
    where the tolerance is exceeded the two must be neighbouring storage values, and such rounding
    flips must stay rare (under 0.5 % of the elements)."""
    dtype = got.dtype
    got, want = got.float().cpu(), want.float().cpu()
    assert not torch.isnan(got).any(), f"{what}: NaN in the output"
    if want_f32 is not None:
        ref = want_f32.float()
        live = ~torch.isnan(ref)  # rows of empty sequences are not produced
        err = (got - ref).abs()[live]
        bound = (ATOL + RTOL * ref.abs())[live]
        worst = (err - bound).max().item() if err.numel() else 0.0
        assert worst <= 0, f"{what}: vs unrounded oracle, max abs err {err.max().item():.4g}, over the bound by {worst:.4g}"
    err = (got - want).abs()
    over = err > ATOL + RTOL * want.abs()
    if over.any():
        flips = over & (err <= 1.001 * ulp_of(dtype, torch.maximum(got.abs(), want.abs())))
        assert torch.equal(flips, over), (
            f"{what}: max abs err {err.max().item():.4g} exceeds the tolerance by more than a rounding flip")
        assert want_f32 is not None, f"{what}: tolerance exceeded and no unrounded oracle value to arbitrate"
        assert flips.float().mean().item() < 5e-3, f"{what}: {int(flips.sum())} rounding flips"
        print(f"{what}: {int(flips.sum())} of {flips.numel()} elements differ from the rounded oracle by one "
              f"{dtype} step (rounding flip); all are within tolerance of its unrounded value", flush=True)


def to_device(inp):
    return [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens)]


def oracle_of(oracle, inp, **kw):
    return oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                  num_threads=ORACLE_THREADS, **kw)


def run_case(gpu_handle, oracle, inp, alibi=None):
    q, k, v, bt, sl = to_device(inp)
    alibi_dev = alibi.to(DEV) if alibi is not None else None
    print(f"case {inp.config.name} B={q.shape[0]} H={q.shape[1]} Hkv={k.shape[1]} D={q.shape[2]} "
          f"bs={k.shape[2]} dtype={q.dtype} lens[:4]={inp.seq_lens[:4].tolist()}", flush=True)
    got = run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale, alibi=alibi_dev)
    want, want_f32 = oracle_of(oracle, inp, alibi_slopes=alibi, return_fp32=True)
    assert_close(got, want, inp.config.name, want_f32)
    return got, want


def custom(name, dtype, B, H, Hkv, D, bs, lo, hi, seed, **kw):
    return workloads.DecodeConfig(name, dtype, B, H, Hkv, D, bs, lo, hi, seed=seed, **kw)


# ---- the benchmark configurations -------------------------------------------------------------------

@pytest.mark.parametrize("schedule", [None, "balanced"], ids=["default_schedule", "balanced"])
def test_c1_plumbing_mha_against_oracle_and_committed_fixture(gpu_handle, oracle, monkeypatch, schedule):
    """c1 under the schedule the library picks for it by itself (a small job: fixed partitions) and under the
    work-equalising one."""
    if schedule is None:
        monkeypatch.delenv("INFINIOP_AMD_PA_SCHEDULE", raising=False)
    inp = workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c1_plumbing_mha"])
    got, _ = run_case(gpu_handle, oracle, inp)
    from pathlib import Path
    fixture = torch.from_numpy(np.load(Path(__file__).parent / "golden" / "c1_plumbing_mha_expected_f64.npy"))
    assert_close(got, fixture, "c1 vs float64 fixture")


def test_c2_llama3_8b_full_size(gpu_handle, oracle):
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c2_llama3_8b_b32"]))


def test_c3_long_context_peaked_softmax_full_size(gpu_handle, oracle):
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c3_long_context"]))


def test_c4_70b_share_full_size(gpu_handle, oracle):
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c4_70b_share_b128"]))


# ---- the reference's own test list -------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(
    "B,H,Hkv,D,bs,max_len",
    [
        # test/infiniop/paged_attention.py:95-105 (the MLA 576/512 row is covered below)
        (1, 1, 1, 128, 16, 1024),
        (4, 40, 40, 128, 16, 1024),
        (6, 40, 40, 128, 16, 1024),
        (3, 8, 8, 128, 16, 1024),
        (3, 8, 8, 64, 16, 1024),
        (8, 64, 8, 128, 16, 2048),
        (1, 16, 16, 192, 16, 256),
        (1, 16, 16, 576, 16, 256),
    ],
)
def test_reference_test_shapes(gpu_handle, oracle, dtype, B, H, Hkv, D, bs, max_len):
    cfg = custom(f"ref_{B}_{H}_{Hkv}_{D}", dtype, B, H, Hkv, D, bs, 1, max_len - 1, seed=7 * B + H + D)
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(cfg))


@pytest.mark.parametrize("schedule", [None, "balanced"], ids=["default_schedule", "balanced"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(
    "B,H,Hkv,D,bs,max_len,Dv",
    [
        # test/infinicore/ops/paged_attention.py:22-38, literally: (num_seqs, num_heads, num_kv_heads, head_size,
        # block_size, max_seq_len[, value_size]); lengths are drawn from [1, max_seq_len) as that test does (:71)
        (1, 1, 1, 128, 16, 15, 0),
        (4, 40, 40, 128, 16, 1024, 0),
        (6, 40, 40, 128, 16, 1024, 0),
        (3, 8, 8, 128, 16, 1024, 0),
        (3, 8, 8, 64, 16, 1024, 0),
        (8, 64, 8, 128, 16, 2048, 0),
        (1, 24, 4, 256, 16, 32, 0),
        (1, 12, 2, 256, 16, 32, 0),
        (1, 6, 1, 256, 16, 32, 0),
        (1, 16, 1, 576, 16, 32, 512),
    ],
)
def test_reference_framework_test_shapes(gpu_handle, oracle, monkeypatch, dtype, B, H, Hkv, D, bs, max_len, Dv, schedule):
    """The shape list of the reference's framework-level test (groups of 6 query heads at head 256, a sequence
    shorter than one page, the latent-attention wrapper case), under the schedule the library picks by itself
    and under the work-equalising one (which the latent shape does not have: it runs its own kernels twice)."""
    if schedule is None:
        monkeypatch.delenv("INFINIOP_AMD_PA_SCHEDULE", raising=False)
    cfg = custom(f"fw_{B}_{H}_{Hkv}_{D}_{max_len}", dtype, B, H, Hkv, D, bs, 1, max_len - 1, seed=11 * B + H + D + max_len,
                 value_size=Dv)
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(cfg))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mla_key_576_value_512(gpu_handle, oracle, dtype):
    """test/infiniop/paged_attention.py:108: (1, 16, 1, 576, 16, 256, value_size 512)."""
    rng = np.random.default_rng(21)
    B, H, Hkv, D, Dv, bs, L = 1, 16, 1, 576, 512, 16, 201
    nb = (L + bs - 1) // bs
    q = torch.from_numpy(rng.standard_normal((B, H, D), dtype=np.float32)).to(dtype)
    k = torch.from_numpy(rng.standard_normal((nb, Hkv, bs, D), dtype=np.float32)).to(dtype)
    v = torch.from_numpy(rng.standard_normal((nb, Hkv, bs, Dv), dtype=np.float32)).to(dtype)
    bt = torch.from_numpy(rng.permutation(nb).astype(np.int64)).view(1, nb)
    sl = torch.tensor([L], dtype=torch.int64)
    scale = 1.0 / D ** 0.5
    got = run_paged_attention(gpu_handle, q.to(DEV), k.to(DEV), v.to(DEV), bt.to(DEV), sl.to(DEV), scale)
    assert got.shape == (B, H, Dv)
    assert_close(got, oracle.paged_attention(q, k, v, bt, sl, scale), "mla")


# ---- head sizes of the tiled kernels -------------------------------------------------------------------

@pytest.mark.parametrize("schedule", [None, "grid", "fused"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 192, 256])
def test_tiled_kernels_other_head_sizes(gpu_handle, oracle, monkeypatch, D, dtype, schedule):
    """Head sizes 64 / 192 / 256 on the matrix-core kernels, both schedules (the work-equalising one also with
    the segments merged inside the decode kernel): ragged lengths incl. 1 token and exactly one page, GQA 4,
    long enough that sequences are split and merged."""
    if schedule == "fused":
        monkeypatch.setenv("INFINIOP_AMD_PA_MERGE", "fused")
    elif schedule:
        monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", schedule)
    cfg = custom(f"head{D}_{schedule}", dtype, 6, 16, 4, D, 16, 1, 2500, seed=300 + D)
    inp = workloads.make_decode_inputs(cfg)
    inp.seq_lens[0], inp.seq_lens[1] = 1, 16
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("D", [64, 192, 256])
def test_other_head_sizes_match_the_elementwise_kernel_bit_for_bit_in_layout(gpu_handle, oracle, monkeypatch, D):
    """Every output column lands where the element-wise kernel puts it: V with a distinct constant per
    column makes the expected output that constant, whatever the softmax does."""
    cfg = custom(f"cols{D}", torch.float16, 3, 8, 2, D, 16, 40, 700, seed=310 + D)
    inp = workloads.make_decode_inputs(cfg)
    ramp = (torch.arange(D, dtype=torch.float32) - D / 2) / 8
    inp.v_cache[:] = ramp.to(torch.float16)
    got = run_paged_attention(gpu_handle, *to_device(inp), inp.scale).float().cpu()
    want = ramp.to(torch.float16).float().expand_as(got)
    assert torch.allclose(got, want, atol=2e-3 * float(ramp.abs().max()), rtol=0), (got - want).abs().max()


@pytest.mark.parametrize("D", [64, 256])
def test_other_head_sizes_alibi_groups_pages_and_index_dtypes(gpu_handle, oracle, D):
    cfg = custom(f"mix{D}", torch.bfloat16, 5, 40, 2, D, 64, 1, 1500, seed=320 + D)  # group of 20: two packs per KV head
    inp = workloads.make_decode_inputs(cfg)
    slopes = torch.tensor([2.0 ** (-(i % 8 + 1)) for i in range(40)], dtype=torch.float32)
    q, k, v, bt, sl = to_device(inp)
    got = run_paged_attention(gpu_handle, q, k, v, bt.to(torch.int32), sl.to(torch.int32), inp.scale, alibi=slopes.to(DEV))
    want, want_f32 = oracle_of(oracle, inp, alibi_slopes=slopes, return_fp32=True)
    assert_close(got, want, cfg.name, want_f32)


@pytest.mark.parametrize("D", [64, 192, 256])
def test_other_head_sizes_ignore_garbage_beyond_the_sequences(gpu_handle, oracle, D):
    inp = workloads.make_decode_inputs(custom(f"poison{D}", torch.float16, 4, 8, 4, D, 16, 1, 600, seed=330 + D))
    want = oracle_of(oracle, inp)
    k, v = inp.k_cache.clone(), inp.v_cache.clone()
    for s in range(4):
        n = int(inp.seq_lens[s])
        if n % 16:
            page = inp.block_tables[s, (n - 1) // 16]
            k[page, :, n % 16:, :] = float("nan")
            v[page, :, n % 16:, :] = float("nan")
    got = run_paged_attention(gpu_handle, inp.q.to(DEV), k.to(DEV), v.to(DEV), inp.block_tables.to(DEV),
                              inp.seq_lens.to(DEV), inp.scale)
    assert_close(got, want, f"poison{D}")


# ---- latent-attention caches: keys of 576, values of 512 (tiled kernel of its own) -------------------------

def mla(name, dtype, B, H, bs, lo, hi, seed, **kw):
    return workloads.DecodeConfig(name, dtype, B, H, 1, 576, bs, lo, hi, seed=seed, value_size=512, **kw)


@pytest.fixture(params=[None, "narrow", "wide", "rows", "wide128"], ids=["auto", "narrow", "wide", "rows", "wide128"])
def latent_kernel(request, monkeypatch):
    """The latent-attention kernels: 16 query heads per workgroup of two wavefronts ("narrow"); tiles shared through LDS
    ("wide": a workgroup of eight wavefronts for a single chunk of 16 heads, otherwise four chunks per workgroup with
    a score and a value wavefront each; "rows": a wavefront per chunk, four per workgroup, or eight with "wide128").
    Left alone, more than 16 heads per KV head and small batches take the wide ones."""
    if request.param:
        monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_KERNEL", "wide" if request.param == "wide128" else request.param)
        if request.param != "narrow":
            monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_HEADS", "128" if request.param == "wide128" else "64")
    return request.param


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H", [16, 128, 20, 48, 80])
def test_mla_ragged_batches(gpu_handle, oracle, dtype, H, latent_kernel):
    """Ragged lengths incl. 1 token and exactly one page, long enough that sequences are split into
    partitions and merged; 16 heads (one chunk of 16), 20 (two chunks, one partly filled), 48 (three: a wide
    workgroup with one slot without heads), 80 (five: two wide workgroups, the second with one chunk) and
    128 (eight)."""
    inp = workloads.make_decode_inputs(mla(f"mla_h{H}", dtype, 5, H, 16, 1, 2500, seed=400 + H))
    inp.seq_lens[0], inp.seq_lens[1] = 1, 16
    got, _ = run_case(gpu_handle, oracle, inp)
    assert got.shape == (5, H, 512)


@pytest.mark.parametrize("partition", [16, 48, 1024])
def test_mla_partition_sizes(gpu_handle, oracle, monkeypatch, partition, latent_kernel):
    """Partitions of one 16-token half tile, of one and a half 32-token tiles, and of the most one page-id
    load covers."""
    monkeypatch.setenv("INFINIOP_AMD_PA_PARTITION", str(partition))
    H = 48 if latent_kernel in ("wide", "rows", "wide128") else 16
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(mla(f"mla_p{partition}", torch.bfloat16, 3, H, 16, 1, 1200, seed=410)))


def test_mla_matches_the_elementwise_kernel_in_layout(gpu_handle, latent_kernel):
    """Every output column lands where the element-wise kernel puts it: V with a distinct constant per
    column makes the expected output that constant, whatever the softmax does. Short sequences (written by the
    decode kernel) and long ones (merged from partitions)."""
    inp = workloads.make_decode_inputs(mla("mla_cols", torch.float16, 4, 16, 16, 40, 1500, seed=420))
    inp.seq_lens[0] = 33
    ramp = (torch.arange(512, dtype=torch.float32) - 256) / 16
    inp.v_cache[:] = ramp.to(torch.float16)
    got = run_paged_attention(gpu_handle, *to_device(inp), inp.scale).float().cpu()
    want = ramp.to(torch.float16).float().expand_as(got)
    assert torch.allclose(got, want, atol=2e-3 * float(ramp.abs().max()), rtol=0), (got - want).abs().max()


def test_mla_alibi_pages_of_64_and_int32_indices(gpu_handle, oracle, latent_kernel):
    inp = workloads.make_decode_inputs(mla("mla_mix", torch.bfloat16, 4, 32, 64, 1, 1500, seed=430))
    slopes = torch.tensor([2.0 ** (-(i % 8 + 1)) for i in range(32)], dtype=torch.float32)
    q, k, v, bt, sl = to_device(inp)
    got = run_paged_attention(gpu_handle, q, k, v, bt.to(torch.int32), sl.to(torch.int32), inp.scale, alibi=slopes.to(DEV))
    want, want_f32 = oracle_of(oracle, inp, alibi_slopes=slopes, return_fp32=True)
    assert_close(got, want, "mla_mix", want_f32)


def test_mla_ignores_garbage_beyond_the_sequences(gpu_handle, oracle, latent_kernel):
    inp = workloads.make_decode_inputs(mla("mla_poison", torch.float16, 4, 16, 16, 1, 600, seed=440))
    want = oracle_of(oracle, inp)
    k, v = inp.k_cache.clone(), inp.v_cache.clone()
    for s in range(4):
        n = int(inp.seq_lens[s])
        if n % 16:
            page = inp.block_tables[s, (n - 1) // 16]
            k[page, :, n % 16:, :] = float("nan")
            v[page, :, n % 16:, :] = float("nan")
    got = run_paged_attention(gpu_handle, inp.q.to(DEV), k.to(DEV), v.to(DEV), inp.block_tables.to(DEV),
                              inp.seq_lens.to(DEV), inp.scale)
    assert_close(got, want, "mla_poison")


def test_mla_padded_cache_rows(gpu_handle, oracle, latent_kernel):
    """K and V rows that are not packed (views into wider pools): row strides of 640 and 576 elements."""
    inp = workloads.make_decode_inputs(mla("mla_strided", torch.bfloat16, 3, 16, 16, 1, 900, seed=450))
    nb = inp.k_cache.shape[0]
    k_pool = torch.full((nb, 1, 16, 640), float("nan"), dtype=torch.bfloat16)
    v_pool = torch.full((nb, 1, 16, 576), float("nan"), dtype=torch.bfloat16)
    k_pool[..., :576] = inp.k_cache
    v_pool[..., :512] = inp.v_cache
    got = run_paged_attention(gpu_handle, inp.q.to(DEV), k_pool.to(DEV)[..., :576], v_pool.to(DEV)[..., :512],
                              inp.block_tables.to(DEV), inp.seq_lens.to(DEV), inp.scale)
    want, want_f32 = oracle_of(oracle, inp, return_fp32=True)
    assert_close(got, want, "mla_strided", want_f32)


# ---- heads of 576 with values of 576 (test/infiniop/paged_attention.py:106): the two-wavefront kernel of the latent
# shape with 288 value columns per wavefront -----------------------------------------------------------------------

def head576(name, dtype, B, H, Hkv, bs, lo, hi, seed, **kw):
    return workloads.DecodeConfig(name, dtype, B, H, Hkv, 576, bs, lo, hi, seed=seed, **kw)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,Hkv", [(16, 16), (20, 1), (40, 2)])
def test_head_576_with_values_of_576(gpu_handle, oracle, tmp_path, dtype, H, Hkv):
    """One head per KV head (the reference's row), a group of 20 (two chunks of 16, one partly filled) and two KV heads;
    lengths of one token, one page and enough for several partitions. The plan takes the tiled kernel."""
    from test_decode_plan import build_probe
    inp = workloads.make_decode_inputs(head576(f"h576_{H}_{Hkv}", dtype, 4, H, Hkv, 16, 1, 2500, seed=900 + H))
    inp.seq_lens[0], inp.seq_lens[1] = 1, 16
    plan = build_probe(tmp_path)(4, H, Hkv, 576, 16, inp.block_tables.shape[1], num_blocks=inp.k_cache.shape[0])
    assert plan["tiled"] == 1 and plan["latent_wide"] == 0 and plan["max_partitions"] > 1
    got, _ = run_case(gpu_handle, oracle, inp)
    assert got.shape == (4, H, 576)


@pytest.mark.parametrize("partition", [16, 48, 1024])
def test_head_576_partition_sizes(gpu_handle, oracle, monkeypatch, partition):
    monkeypatch.setenv("INFINIOP_AMD_PA_PARTITION", str(partition))
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(head576(f"h576_p{partition}", torch.bfloat16, 3, 16, 4, 16, 1, 1200, seed=910)))


def test_head_576_matches_the_elementwise_kernel_in_layout(gpu_handle):
    """Every one of the 576 output columns lands in its place (see the latent-attention test of the same name), for
    sequences written by the decode kernel and for merged ones."""
    inp = workloads.make_decode_inputs(head576("h576_cols", torch.float16, 4, 16, 2, 16, 40, 1500, seed=920))
    inp.seq_lens[0] = 33
    ramp = (torch.arange(576, dtype=torch.float32) - 288) / 16
    inp.v_cache[:] = ramp.to(torch.float16)
    got = run_paged_attention(gpu_handle, *to_device(inp), inp.scale).float().cpu()
    want = ramp.to(torch.float16).float().expand_as(got)
    assert torch.allclose(got, want, atol=2e-3 * float(ramp.abs().max()), rtol=0), (got - want).abs().max()


def test_head_576_alibi_pages_of_64_int32_indices_and_garbage_beyond_the_sequences(gpu_handle, oracle):
    inp = workloads.make_decode_inputs(head576("h576_mix", torch.bfloat16, 4, 32, 2, 64, 1, 1500, seed=930))
    slopes = torch.tensor([2.0 ** (-(i % 8 + 1)) for i in range(32)], dtype=torch.float32)
    want, want_f32 = oracle_of(oracle, inp, alibi_slopes=slopes, return_fp32=True)
    k, v = inp.k_cache.clone(), inp.v_cache.clone()
    for s in range(4):
        n = int(inp.seq_lens[s])
        if n % 64:
            page = inp.block_tables[s, (n - 1) // 64]
            k[page, :, n % 64:, :] = float("nan")
            v[page, :, n % 64:, :] = float("nan")
    got = run_paged_attention(gpu_handle, inp.q.to(DEV), k.to(DEV), v.to(DEV), inp.block_tables.to(DEV).to(torch.int32),
                              inp.seq_lens.to(DEV).to(torch.int32), inp.scale, alibi=slopes.to(DEV))
    assert_close(got, want, "h576_mix", want_f32)


@pytest.mark.parametrize("workload", ["m1_mla_16_heads_b32", "m2_mla_128_heads_b32"])
def test_mla_full_size_against_oracle(gpu_handle, oracle, workload):
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(workloads.DECODE_CONFIGS[workload]))


def test_mla_empty_and_negative_lengths_in_the_per_call_plan(gpu_handle, oracle):
    """The 64-head kernel numbers its units from the lengths it reads itself: sequences without tokens get
    none, and their output rows stay untouched."""
    inp = workloads.make_decode_inputs(mla("mla_empty", torch.float16, 7, 48, 16, 1, 2000, seed=460))
    inp.seq_lens[0], inp.seq_lens[3], inp.seq_lens[6] = 0, -7, 0
    q, k, v, bt, sl = to_device(inp)
    out = torch.full((7, 48, 512), 7.0, dtype=torch.float16, device=DEV)
    run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale, out=out)
    want = torch.full((7, 48, 512), 7.0, dtype=torch.float16)
    oracle_of(oracle, inp, out=want)
    for s in (0, 3, 6):
        assert torch.all(out[s] == 7)
    assert_close(out, want, "mla_empty")


def test_mla_per_call_plan_is_in_use(gpu_handle, tmp_path):
    """The 64-head kernel chooses its partition size per call from the actual lengths and leaves it in the
    workspace for the merge kernel (first word behind the partial results): after a call that word holds a
    size the plan can produce, not the bytes the workspace was filled with."""
    from test_decode_plan import build_probe

    inp = workloads.make_decode_inputs(mla("mla_planned", torch.bfloat16, 8, 128, 16, 600, 2500, seed=465))
    q, k, v, bt, sl = to_device(inp)
    out = torch.zeros((8, 128, 512), dtype=torch.bfloat16, device=DEV)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    assert status == 0
    size = workspace_size_attention(op)
    ws = torch.full((size,), 0xFF, dtype=torch.uint8, device=DEV)
    assert ws.data_ptr() % 256 == 0
    L.check_error(L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size, ptr(out), ptr(q), ptr(k), ptr(v), ptr(bt), ptr(sl), None, None))
    torch.cuda.synchronize()
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))
    plan = build_probe(tmp_path)(8, 128, 1, 576, 16, bt.shape[1], value_size=512, num_blocks=k.shape[0])
    assert plan["latent_wide"] and plan["workspace_bytes"] == size
    offset = plan["acc_bytes"] + 2 * plan["ml_bytes"]
    chosen = int(ws[offset:offset + 4].view(torch.int32).item())
    assert 128 <= chosen <= 1024 and chosen % 64 == 0, chosen


def test_mla_remembered_partition_search(gpu_handle, oracle, tmp_path):
    """The search for the partition size is remembered in the workspace (a hash of the lengths and the shape with the
    size found) and skipped by later calls on the same lengths: such calls reproduce the first one bit for bit, a
    call on other lengths through the same workspace searches again and is right, and going back is right again."""
    from test_decode_plan import build_probe

    inp = workloads.make_decode_inputs(mla("mla_remember", torch.bfloat16, 24, 128, 16, 600, 2500, seed=466))
    q, k, v, bt, sl = to_device(inp)
    out = torch.zeros((24, 128, 512), dtype=torch.bfloat16, device=DEV)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    assert status == 0
    size = workspace_size_attention(op)
    ws = torch.full((size,), 0xFF, dtype=torch.uint8, device=DEV)
    plan = build_probe(tmp_path)(24, 128, 1, 576, 16, bt.shape[1], value_size=512, num_blocks=k.shape[0])
    offset = plan["acc_bytes"] + 2 * plan["ml_bytes"]

    def call():
        out.zero_()
        L.check_error(L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size, ptr(out), ptr(q), ptr(k), ptr(v), ptr(bt), ptr(sl), None, None))
        torch.cuda.synchronize()
        chosen = int(ws[offset:offset + 4].view(torch.int32).item())
        word = int(ws[offset + 8:offset + 16].view(torch.int64).item()) & 0xFFFFFFFFFFFFFFFF
        return out.clone(), chosen, word

    first, chosen_a, word_a = call()
    assert chosen_a > plan["partition_tokens"], "the case must make the kernel search beyond the planned size"
    assert chosen_a == plan["partition_tokens"] + 64 * (word_a & 0xFF)
    assert_close(first.cpu(), oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale), "mla_remember")
    again, chosen, word = call()
    assert (chosen, word) == (chosen_a, word_a) and torch.equal(again.view(torch.int16), first.view(torch.int16))
    long_lens = inp.seq_lens.clone()
    inp.seq_lens[:] = inp.seq_lens - 37  # other lengths under the same block table, still too many partitions for one round
    sl.copy_(inp.seq_lens)
    other, chosen_b, word_b = call()
    assert word_b != word_a and chosen_b == plan["partition_tokens"] + 64 * (word_b & 0xFF)
    assert_close(other.cpu(), oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale), "mla_remember_other")
    inp.seq_lens[:] = long_lens
    sl.copy_(long_lens)
    back, chosen, word = call()
    assert (chosen, word) == (chosen_a, word_a) and torch.equal(back.view(torch.int16), first.view(torch.int16))
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


def test_mla_batches_that_take_128_heads_per_workgroup_by_themselves(gpu_handle, oracle, tmp_path):
    """From 48 sequences x KV heads on, more than 64 query heads per KV head share one workgroup of eight wavefronts
    (no knob set): 50 ragged sequences of 128 and of 80 heads (five chunks: three wavefronts without heads)."""
    from test_decode_plan import build_probe

    for H in (128, 80):
        inp = workloads.make_decode_inputs(mla(f"mla_b50_h{H}", torch.bfloat16, 50, H, 16, 1, 700, seed=475 + H))
        plan = build_probe(tmp_path)(50, H, 1, 576, 16, inp.block_tables.shape[1], value_size=512, num_blocks=inp.k_cache.shape[0])
        assert plan["latent_wide"] and plan["latent_chunks"] == 8
        run_case(gpu_handle, oracle, inp)


def test_mla_more_sequences_than_the_per_call_plan_handles(gpu_handle, oracle):
    """More than 256 sequences: fixed partitions on the three-dimensional grid."""
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(mla("mla_b300", torch.bfloat16, 300, 32, 16, 1, 400, seed=470)))


def test_mla_sequences_that_fit_one_partition_need_no_workspace(gpu_handle, oracle):
    inp = workloads.make_decode_inputs(mla("mla_short", torch.float16, 5, 64, 16, 1, 100, seed=480))
    q, k, v, bt, sl = to_device(inp)
    out = torch.zeros((5, 64, 512), dtype=torch.float16, device=DEV)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    assert status == 0 and workspace_size_attention(op) == 0
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("B,lo,hi", [(1, 2100, 2100), (4, 512, 4096), (16, 512, 4096)])
def test_default_schedule_choice(gpu_handle, oracle, monkeypatch, B, lo, hi):
    """No knob set: one sequence and four ragged ones take the fixed partitions (small job), sixteen the
    work-equalising schedule; all must agree with the oracle."""
    monkeypatch.delenv("INFINIOP_AMD_PA_SCHEDULE", raising=False)
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(custom(f"default_b{B}", torch.bfloat16, B, 32, 8, 128, 16, lo, hi, seed=500 + B)))


# ---- every kernel and schedule against the same oracle ---------------------------------------------

@pytest.mark.parametrize("kernel,schedule", [("generic", None), (None, "grid"), (None, None), (None, "fused")])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_kernels_and_schedules_agree_with_oracle(gpu_handle, oracle, monkeypatch, kernel, schedule, dtype):
    if kernel:
        monkeypatch.setenv("INFINIOP_AMD_PA_KERNEL", kernel)
    if schedule == "fused":  # the work-equalising schedule with the segments merged inside the decode kernel
        monkeypatch.setenv("INFINIOP_AMD_PA_MERGE", "fused")
    elif schedule:
        monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", schedule)
    cfg = custom(f"ragged_{kernel}_{schedule}", dtype, 6, 32, 8, 128, 16, 1, 3000, seed=5)
    inp = workloads.make_decode_inputs(cfg)
    inp.seq_lens[0], inp.seq_lens[1] = 1, 16  # shortest possible and exactly one page
    run_case(gpu_handle, oracle, inp)


def climbing_keys(inp, step_log2=0.25, jump_every=200, jump_log2=12.0):
    """Overwrites K so that the scores of every query head climb along the sequence: by step_log2 (in
    powers of two of the softmax weight) per token, plus jump_log2 at every jump_every-th token. The
    running maximum then moves in every tile, by less than a tile's rescaling threshold most of the time
    and by much more at the jumps."""
    cfg = inp.config
    rng = np.random.default_rng(cfg.seed + 1)
    direction = torch.from_numpy(rng.standard_normal((cfg.num_kv_heads, cfg.head_size)).astype(np.float32))
    direction /= direction.norm(dim=1, keepdim=True)
    group = cfg.num_heads // cfg.num_kv_heads
    # every query head points along its KV head's direction: score = |q| * a(t) * scale
    q_norm = 4.0
    inp.q[:] = (direction.repeat_interleave(group, dim=0)[None] * q_norm).to(cfg.dtype).expand_as(inp.q)
    per_unit = q_norm * inp.scale * 1.4426950408889634  # log2 of the weight per unit of a(t)
    for s in range(cfg.num_seqs):
        n = int(inp.seq_lens[s])
        t = torch.arange(n, dtype=torch.float32)
        a = (step_log2 * t + jump_log2 * torch.floor(t / jump_every)) / per_unit
        a -= a.mean()
        rows = a[:, None, None] * direction[None] + 0.05 * torch.from_numpy(
            rng.standard_normal((n, cfg.num_kv_heads, cfg.head_size)).astype(np.float32))
        pages = inp.block_tables[s, torch.arange(n) // cfg.block_size]
        inp.k_cache[pages, :, torch.arange(n) % cfg.block_size] = rows.to(cfg.dtype)
    return inp


@pytest.mark.parametrize("schedule", [None, "grid"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_scores_that_climb_along_the_sequence(gpu_handle, oracle, monkeypatch, dtype, schedule):
    if schedule:
        monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", schedule)
    inp = climbing_keys(workloads.make_decode_inputs(custom(f"climb_{schedule}", dtype, 4, 32, 8, 128, 16, 300, 1500, seed=71)))
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_mla_scores_that_climb_along_the_sequence(gpu_handle, oracle, dtype, latent_kernel):
    inp = climbing_keys(workloads.make_decode_inputs(mla("mla_climb", dtype, 3, 16, 16, 300, 1200, seed=72)))
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("partition", [16, 64, 1024])
def test_grid_schedule_partition_sizes(gpu_handle, oracle, monkeypatch, partition):
    monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", "grid")
    monkeypatch.setenv("INFINIOP_AMD_PA_PARTITION", str(partition))
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(custom("part", torch.bfloat16, 4, 16, 4, 128, 16, 1, 2500, seed=3)))


@pytest.mark.parametrize("heads,D,Dv", [(16, 128, 0), (16, 576, 512), (48, 576, 512)])
def test_partitions_of_large_pages_stay_inside_one_page_id_load(gpu_handle, oracle, monkeypatch, heads, D, Dv):
    """Pages of 64 tokens and a requested partition of 4080 tokens (not a multiple of the page): the plan rounds
    it to whole pages, so that partition 1 of a sequence of more than 8200 tokens does not start inside a page
    and need a 65th block-table entry. Fixed partitions, all three tiled kernel families."""
    monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", "grid")
    monkeypatch.setenv("INFINIOP_AMD_PA_PARTITION", "4080")
    cfg = custom(f"bigpages_{heads}_{D}", torch.bfloat16, 2, heads, 1 if D == 576 else 4, D, 64, 8300, 8900, seed=83,
                 value_size=Dv)
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(cfg))


@pytest.mark.parametrize("waves_per_cu", [1, 2, 8, 16])
def test_balanced_schedule_any_piece_count(gpu_handle, oracle, monkeypatch, waves_per_cu):
    monkeypatch.setenv("INFINIOP_AMD_PA_WAVES_PER_CU", str(waves_per_cu))
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(custom("pieces", torch.float16, 9, 32, 8, 128, 16, 1, 1800, seed=13)))


def test_many_short_sequences_per_piece(gpu_handle, oracle):
    """Hundreds of sequences of a few tokens: every wavefront's piece spans many sequences."""
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(custom("short", torch.bfloat16, 700, 8, 2, 128, 16, 1, 40, seed=17)))


def test_more_sequences_than_the_balanced_schedule_handles(gpu_handle, oracle):
    """Above 1024 sequences the plan falls back to the plain grid of partitions."""
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(custom("wide", torch.float16, 1100, 4, 4, 128, 16, 1, 70, seed=19)))


@pytest.mark.parametrize("H,Hkv", [(40, 2), (32, 1), (24, 8)])
def test_query_groups_larger_than_one_wavefront_packs(gpu_handle, oracle, H, Hkv):
    """Groups of 20, 32 and 3 query heads per KV head (more than 16 are split into chunks)."""
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(custom("groups", torch.bfloat16, 3, H, Hkv, 128, 16, 10, 900, seed=H)))


@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256, 8, 48])
def test_page_sizes(gpu_handle, oracle, bs):
    """Powers of two from 16 use the tiled kernel; 8 and 48 take the element-wise one."""
    run_case(gpu_handle, oracle, workloads.make_decode_inputs(custom(f"bs{bs}", torch.float16, 4, 8, 2, 128, bs, 1, 1500, seed=bs)))


@pytest.mark.parametrize("index_dtype", [torch.int32, torch.uint32, torch.int64])
def test_index_dtypes(gpu_handle, oracle, index_dtype):
    inp = workloads.make_decode_inputs(custom("idx", torch.bfloat16, 5, 16, 4, 128, 16, 1, 700, seed=23))
    q, k, v, bt, sl = to_device(inp)
    got = run_paged_attention(gpu_handle, q, k, v, bt.to(index_dtype), sl.to(index_dtype), inp.scale)
    assert_close(got, oracle_of(oracle, inp), f"index {index_dtype}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kernel", [None, "generic"])
def test_alibi(gpu_handle, oracle, monkeypatch, dtype, kernel):
    """No reference test enables ALiBi; the expected value is the oracle's, itself pinned against the
    float64 formulation with bias."""
    if kernel:
        monkeypatch.setenv("INFINIOP_AMD_PA_KERNEL", kernel)
    inp = workloads.make_decode_inputs(custom("alibi", dtype, 4, 16, 4, 128, 16, 1, 900, seed=29))
    slopes = torch.tensor([2.0 ** (-8.0 * (i + 1) / 16) for i in range(16)], dtype=torch.float32)
    got, want = run_case(gpu_handle, oracle, inp, alibi=slopes)
    assert not torch.equal(want, oracle_of(oracle, inp))


# ---- a seeded sweep over everything at once ------------------------------------------------------------

@pytest.mark.parametrize("seed", range(int(os.environ.get("INFINICORE_AMD_TEST_SWEEP_SEEDS", "40"))))
def test_random_shapes_schedules_and_dtypes(gpu_handle, oracle, monkeypatch, seed):
    """Every knob drawn at random from one seed: head size (tiled sizes, 576 / 512 and 576 / 576), group size, page size,
    batch, lengths (with empty sequences), dtype, index dtype, ALiBi, schedule and merge mode. The cases above
    vary one thing at a time; this one guards the combinations."""
    rng = np.random.default_rng(1000 + seed)
    D, Dv = [(64, 0), (128, 0), (128, 0), (192, 0), (256, 0), (576, 512), (576, 512), (576, 576)][rng.integers(0, 8)]
    Hkv = int(rng.choice([1, 1, 2])) if D == 576 else int(rng.choice([1, 2, 4, 8]))
    group = int(rng.choice([1, 2, 3, 4, 7, 16, 20])) if D != 576 else int(rng.choice([1, 4, 16, 20, 48, 64, 100, 128]))
    bs = int(rng.choice([8, 16, 16, 32, 64, 128])) if D != 576 else int(rng.choice([16, 32, 64]))
    B = int(rng.choice([1, 2, 5, 17, 40])) if D != 576 else int(rng.choice([1, 2, 5, 9]))
    hi = int(rng.choice([40, 300, 1500, 5000])) if D != 576 else int(rng.choice([40, 300, 1500]))
    dtype = [torch.float16, torch.bfloat16][rng.integers(0, 2)]
    index_dtype = [torch.int64, torch.int32, torch.uint32][rng.integers(0, 3)]
    schedule = [None, "balanced", "grid"][rng.integers(0, 3)]
    merge = ["kernel", "fused"][rng.integers(0, 2)]
    latent_kernel = [None, "narrow", "wide", "rows"][rng.integers(0, 4)]
    use_alibi = bool(rng.integers(0, 2))
    monkeypatch.delenv("INFINIOP_AMD_PA_SCHEDULE", raising=False)
    if schedule:
        monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", schedule)
    monkeypatch.setenv("INFINIOP_AMD_PA_MERGE", merge)
    monkeypatch.delenv("INFINIOP_AMD_PA_LATENT_KERNEL", raising=False)
    if latent_kernel:
        monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_KERNEL", latent_kernel)
    H = Hkv * group
    inp = workloads.make_decode_inputs(custom(f"sweep{seed}", dtype, B, H, Hkv, D, bs, 1, hi, seed=700 + seed,
                                              value_size=Dv, spare_block_fraction=0.25))
    lens = inp.seq_lens.clone()
    if B > 2:
        lens[int(rng.integers(0, B))] = 0  # an empty sequence in the middle of the batch
    slopes = torch.tensor(rng.uniform(0.001, 0.3, H), dtype=torch.float32) if use_alibi else None
    print(f"sweep {seed}: D={D}/{Dv or D} H={H}/{Hkv} bs={bs} B={B} hi={hi} {dtype} {index_dtype} schedule={schedule} "
          f"merge={merge} latent={latent_kernel} alibi={use_alibi}", flush=True)
    q, k, v, bt, _ = to_device(inp)
    out = torch.full((B, H, Dv or D), 7.0, dtype=dtype, device=DEV)
    got = run_paged_attention(gpu_handle, q, k, v, bt.to(index_dtype), lens.to(index_dtype).to(DEV), inp.scale,
                              alibi=slopes.to(DEV) if use_alibi else None, out=out)
    want, want_f32 = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, lens, inp.scale,
                                            alibi_slopes=slopes, num_threads=ORACLE_THREADS, return_fp32=True,
                                            out=torch.full((B, H, Dv or D), 7.0, dtype=dtype))
    assert_close(got, want, f"sweep{seed}", want_f32)


# ---- layouts ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_permuted_pool_and_padded_query_rows(gpu_handle, oracle, dtype):
    """Pool stored [pages, rows, heads, d] and handed over as a permuted view (the layout the
    reference's test/infinicore/ops/paged_caching.py:22-34 exercises); q and out rows padded."""
    inp = workloads.make_decode_inputs(custom("strided", dtype, 4, 16, 4, 128, 16, 1, 1200, seed=31))
    q, k, v, bt, sl = to_device(inp)
    k_perm = k.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    v_perm = v.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    q_pad = torch.zeros(4, 16, 192, dtype=dtype, device=DEV)[:, :, :128]
    q_pad.copy_(q)
    out_pad = torch.zeros(4, 20, 128, dtype=dtype, device=DEV)[:, :16, :]
    assert not k_perm.is_contiguous() and not q_pad.is_contiguous() and not out_pad.is_contiguous()
    got = run_paged_attention(gpu_handle, q_pad, k_perm, v_perm, bt, sl, inp.scale, out=out_pad)
    assert_close(got, oracle_of(oracle, inp), "strided")


def test_unaligned_base_addresses_take_the_elementwise_kernel(gpu_handle, oracle):
    """Operands that start 2 bytes into an allocation cannot be read 16 bytes at a time."""
    inp = workloads.make_decode_inputs(custom("unaligned", torch.float16, 2, 8, 2, 128, 16, 1, 300, seed=37))
    q, k, v, bt, sl = to_device(inp)

    def shifted(t):
        flat = torch.zeros(t.numel() + 1, dtype=t.dtype, device=DEV)
        view = flat[1:].view(t.shape)
        view.copy_(t)
        return view

    got = run_paged_attention(gpu_handle, shifted(q), shifted(k), shifted(v), bt, sl, inp.scale)
    assert_close(got, oracle_of(oracle, inp), "unaligned")


def test_unaligned_operands_of_a_large_job_fit_the_planned_workspace(gpu_handle, oracle):
    """A descriptor planned for the work-equalising schedule sizes the workspace for that schedule; when the
    operands of a call are not 16-byte aligned the element-wise kernel runs on partitions cut to fit it."""
    inp = workloads.make_decode_inputs(custom("unaligned_big", torch.bfloat16, 12, 8, 2, 128, 16, 100, 3000, seed=38))
    q, k, v, bt, sl = to_device(inp)

    def shifted(t):
        flat = torch.zeros(t.numel() + 1, dtype=t.dtype, device=DEV)
        view = flat[1:].view(t.shape)
        view.copy_(t)
        return view

    aligned = run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale)
    got = run_paged_attention(gpu_handle, shifted(q), k, v, bt, sl, inp.scale)
    want, want_f32 = oracle_of(oracle, inp, return_fp32=True)
    assert_close(aligned, want, "aligned", want_f32)
    assert_close(got, want, "unaligned_big", want_f32)


# ---- what must not be read, what must not be written -------------------------------------------------

@pytest.mark.parametrize("schedule", [None, "grid"])
def test_nothing_outside_the_sequences_is_read(gpu_handle, oracle, monkeypatch, schedule):
    """NaN in every row past a sequence's end and in unused pages, garbage in table entries past the
    last needed page and in the workspace: the output must not change."""
    if schedule:
        monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", schedule)
    inp = workloads.make_decode_inputs(custom("poison", torch.bfloat16, 6, 16, 4, 128, 16, 1, 900, seed=41,
                                              spare_block_fraction=0.3))
    want = oracle_of(oracle, inp)
    k, v, bt = inp.k_cache.clone(), inp.v_cache.clone(), inp.block_tables.clone()
    used = torch.zeros(k.shape[0], dtype=torch.bool)
    for s in range(6):
        n = int(inp.seq_lens[s])
        last = (n - 1) // 16
        used[bt[s, :last + 1]] = True
        if n % 16:
            k[bt[s, last], :, n % 16:, :] = float("nan")
            v[bt[s, last], :, n % 16:, :] = float("nan")
        bt[s, last + 1:] = 2 ** 40 + 12345
    k[~used] = float("nan")
    v[~used] = float("nan")
    for fill in (0xFF, 0x01):
        got = run_paged_attention(gpu_handle, inp.q.to(DEV), k.to(DEV), v.to(DEV), bt.to(DEV), inp.seq_lens.to(DEV),
                                  inp.scale, workspace_fill=fill)
        assert_close(got, want, f"poison fill={fill:#x}")


@pytest.mark.parametrize("schedule", [None, "grid"])
def test_empty_sequences_leave_their_output_rows_untouched(gpu_handle, oracle, monkeypatch, schedule):
    """seq_len <= 0 writes nothing (reference kernel_v2.cuh:164-167)."""
    if schedule:
        monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", schedule)
    inp = workloads.make_decode_inputs(custom("empty", torch.float16, 6, 8, 2, 128, 16, 1, 600, seed=43))
    inp.seq_lens[0] = 0
    inp.seq_lens[3] = -7
    inp.seq_lens[5] = 0
    q, k, v, bt, sl = to_device(inp)
    out = torch.full((6, 8, 128), 7.0, dtype=torch.float16, device=DEV)
    run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale, out=out)
    want = torch.full((6, 8, 128), 7.0, dtype=torch.float16)
    oracle_of(oracle, inp, out=want)
    for s in (0, 3, 5):
        assert torch.all(out[s] == 7)
    assert_close(out, want, "empty")


def test_all_sequences_empty(gpu_handle):
    inp = workloads.make_decode_inputs(custom("allempty", torch.float16, 3, 8, 2, 128, 16, 1, 50, seed=47))
    q, k, v, bt, sl = to_device(inp)
    out = torch.full((3, 8, 128), 3.0, dtype=torch.float16, device=DEV)
    run_paged_attention(gpu_handle, q, k, v, bt, torch.zeros_like(sl), inp.scale, out=out)
    assert torch.all(out == 3)


# ---- descriptor life cycle ----------------------------------------------------------------------------

def test_one_descriptor_many_calls_with_changing_lengths(gpu_handle, oracle):
    """Lengths and tables live in device memory and change from call to call (every decode step); the
    descriptor and workspace are created once. Also runs on a stream of the runtime's own."""
    inp = workloads.make_decode_inputs(custom("steps", torch.bfloat16, 8, 32, 8, 128, 16, 100, 2000, seed=53))
    q, k, v, bt, sl = to_device(inp)
    out = torch.zeros_like(q)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    assert status == 0
    size = workspace_size_attention(op)
    ws = torch.empty(size, dtype=torch.uint8, device=DEV)
    stream = ctypes.c_void_p()
    L.check_error(L.LIBINFINIRT.infinirtStreamCreate(ctypes.byref(stream)))
    torch.cuda.synchronize()
    for step in range(4):
        lens = torch.clamp(inp.seq_lens - 97 * step, min=1)
        sl.copy_(lens)
        torch.cuda.synchronize()
        L.check_error(L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size, ptr(out), ptr(q), ptr(k), ptr(v), ptr(bt),
                                                           ptr(sl), None, stream))
        L.check_error(L.LIBINFINIRT.infinirtStreamSynchronize(stream))
        want = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, lens, inp.scale,
                                      num_threads=ORACLE_THREADS)
        assert_close(out, want, f"step {step}")
    L.check_error(L.LIBINFINIRT.infinirtStreamDestroy(stream))
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


@pytest.mark.parametrize("merge", ["kernel", "fused"])
@pytest.mark.parametrize("pools", [1, 3])
def test_many_calls_on_one_workspace(gpu_handle, oracle, monkeypatch, pools, merge):
    """One descriptor and workspace, many calls back to back on one or three KV pools, the workspace full of
    random bytes before the first: every call must stay within the tolerance of the oracle. With the segments
    merged by the second kernel and inside the decode kernel (whose flags each call must leave cleared)."""
    monkeypatch.setenv("INFINIOP_AMD_PA_MERGE", merge)
    inp = workloads.make_decode_inputs(custom("adaptive", torch.bfloat16, 16, 32, 8, 128, 16, 200, 2500, seed=91))
    q, k, v, bt, sl = to_device(inp)
    ks, vs = [k] + [k.clone() for _ in range(pools - 1)], [v] + [v.clone() for _ in range(pools - 1)]
    out = torch.zeros_like(q)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    assert status == 0
    size = workspace_size_attention(op)
    ws = torch.empty(size, dtype=torch.uint8, device=DEV).random_(0, 255)
    want, want_f32 = oracle_of(oracle, inp, return_fp32=True)
    for call in range(12):
        out.zero_()
        L.check_error(L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size, ptr(out), ptr(q), ptr(ks[call % pools]),
                                                           ptr(vs[call % pools]), ptr(bt), ptr(sl), None, None))
        torch.cuda.synchronize()
        assert_close(out, want, f"call {call}", want_f32)
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


def test_remembered_first_tiles_never_leak_into_another_batch(gpu_handle, oracle):
    """The work-equalising kernel starts its pipeline with the tiles it guesses from what the previous call left
    in the workspace, and checks the guess against the block table. One descriptor and workspace; between calls
    the pages move (same lengths, another table and pool: every guess names a page that now holds other tokens),
    then the lengths change too, then the first batch returns: every call must match the oracle of its own batch."""
    base = custom("guess_a", torch.bfloat16, 12, 32, 8, 128, 16, 300, 2500, seed=77)
    a = workloads.make_decode_inputs(base)
    moved = workloads.make_decode_inputs(custom("guess_b", torch.bfloat16, 12, 32, 8, 128, 16, 300, 2500, seed=78))
    # same lengths as `a`, the table and pool contents of `moved` where they are long enough: rebuild from a's lengths
    b = workloads.make_decode_inputs(base)
    perm = torch.randperm(b.k_cache.shape[0], generator=torch.Generator().manual_seed(5))
    inverse = torch.empty_like(perm)
    inverse[perm] = torch.arange(perm.numel())
    b.k_cache, b.v_cache = b.k_cache[perm].contiguous(), b.v_cache[perm].contiguous()  # page i now lives at inverse[i]
    b.block_tables = inverse[b.block_tables]
    b.q = moved.q
    q, k, v, bt, sl = to_device(a)
    out = torch.zeros_like(q)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, a.scale)
    assert status == 0
    size = workspace_size_attention(op)
    ws = torch.empty(size, dtype=torch.uint8, device=DEV).random_(0, 255)
    shorter = workloads.make_decode_inputs(base)
    shorter.seq_lens = (shorter.seq_lens * 2) // 3
    for step, inp in enumerate([a, a, b, b, shorter, a, b]):
        qd, kd, vd, btd, sld = to_device(inp)
        out.zero_()
        L.check_error(L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size, ptr(out), ptr(qd), ptr(kd), ptr(vd),
                                                           ptr(btd), ptr(sld), None, None))
        torch.cuda.synchronize()
        want, want_f32 = oracle_of(oracle, inp, return_fp32=True)
        assert_close(out, want, f"step {step}", want_f32)
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 128, 192, 256])
@pytest.mark.parametrize("H,Hkv", [(8, 8), (4, 2), (6, 2), (16, 4), (16, 2)])
def test_merge_inside_the_decode_kernel_at_every_group_size(gpu_handle, oracle, monkeypatch, D, H, Hkv, dtype):
    """The reader of a sequence with one to four heads per KV head (rows spread over all lanes, eight segments per
    round trip) and with eight (a lane group per four heads, four segments per round trip); two long sequences, cut
    into some sixty segments each, next to short ones and an empty one; work-equalising schedule forced (these
    batches are small jobs)."""
    monkeypatch.setenv("INFINIOP_AMD_PA_MERGE", "fused")
    monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", "balanced")
    inp = workloads.make_decode_inputs(custom(f"reader_d{D}_h{H}_{Hkv}", dtype, 6, H, Hkv, D, 16, 1, 300, seed=700 + D + H))
    lens = inp.seq_lens.clone()
    # make_decode_inputs sized the block table for the drawn lengths: draw again with two long sequences
    cfg = custom(f"reader_long_d{D}_h{H}_{Hkv}", dtype, 6, H, Hkv, D, 16, 6000, 9000, seed=701 + D + H)
    inp = workloads.make_decode_inputs(cfg)
    inp.seq_lens[1], inp.seq_lens[2], inp.seq_lens[4], inp.seq_lens[5] = 0, int(lens[2]), 17, int(lens[5])
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("D,B", [(64, 40), (128, 136), (64, 136)])
def test_batches_whose_segments_are_merged_inside_the_decode_kernel_by_default(gpu_handle, oracle, monkeypatch, D, B):
    """No merge knob set: batches of many sequences per piece (and, at head 64, of a few pieces per sequence) are
    merged by the decode kernel itself; they must agree with the oracle like the others, call after call on
    one workspace."""
    monkeypatch.delenv("INFINIOP_AMD_PA_MERGE", raising=False)
    inp = workloads.make_decode_inputs(custom(f"default_merge_d{D}_b{B}", torch.bfloat16, B, 16, 4, D, 16, 1, 700, seed=640 + B + D))
    inp.seq_lens[1], inp.seq_lens[5] = 0, 1
    q, k, v, bt, sl = to_device(inp)
    out = torch.zeros_like(q)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    assert status == 0
    size = workspace_size_attention(op)
    ws = torch.empty(size, dtype=torch.uint8, device=DEV).random_(0, 255)
    want, want_f32 = oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                            num_threads=ORACLE_THREADS, return_fp32=True, out=torch.zeros_like(inp.q))
    for call in range(4):
        out.zero_()
        L.check_error(L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size, ptr(out), ptr(q), ptr(k), ptr(v), ptr(bt),
                                                           ptr(sl), None, None))
        torch.cuda.synchronize()
        assert_close(out, want, f"call {call}", want_f32)
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


@pytest.mark.parametrize("relief", [0, 16, 40, 64])
@pytest.mark.parametrize("D", [64, 128, 192])
def test_uneven_piece_pairs(gpu_handle, oracle, monkeypatch, D, relief):
    """Odd pieces hand a share of their slots to their even neighbours (a fixed share by default where the odd
    accelerator dies stream slower): any share from none to a quarter of a piece must cut the batch into pieces
    that cover every tile exactly once, and tell the merge kernel the right piece range of every sequence."""
    monkeypatch.setenv("INFINIOP_AMD_PA_ODD_RELIEF", str(relief))
    inp = workloads.make_decode_inputs(custom(f"relief{relief}_d{D}", torch.float16, 9, 16, 4, D, 16, 1, 4000, seed=900 + relief))
    inp.seq_lens[0], inp.seq_lens[3] = 1, 0
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("shape", ["head128", "head128_fused_merge", "latent64heads"])
def test_capture_and_replay(gpu_handle, oracle, monkeypatch, shape):
    """The run call allocates nothing and never synchronises, so it can be recorded into a graph;
    every replay (with eager work in between) must reproduce the eager result. The latent-attention case
    plans its units inside the kernel, from the lengths in device memory; with the segments merged inside the
    decode kernel every replay carries the token of the captured call, so each must find the flags cleared."""
    if shape == "head128_fused_merge":
        monkeypatch.setenv("INFINIOP_AMD_PA_MERGE", "fused")
    if shape.startswith("head128"):
        inp = workloads.make_decode_inputs(custom("graph", torch.float16, 6, 32, 8, 128, 16, 50, 1500, seed=59))
    else:
        inp = workloads.make_decode_inputs(mla("graph_latent", torch.bfloat16, 6, 64, 16, 50, 1500, seed=60))
    q, k, v, bt, sl = to_device(inp)
    out = torch.zeros((*q.shape[:2], v.shape[-1]), dtype=q.dtype, device=DEV)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    assert status == 0
    size = workspace_size_attention(op)
    ws = torch.empty(size, dtype=torch.uint8, device=DEV)
    rt = L.LIBINFINIRT
    stream, graph, graph_exec = ctypes.c_void_p(), ctypes.c_void_p(), ctypes.c_void_p()
    L.check_error(rt.infinirtStreamCreate(ctypes.byref(stream)))
    torch.cuda.synchronize()

    def call():
        L.check_error(L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size, ptr(out), ptr(q), ptr(k), ptr(v), ptr(bt),
                                                           ptr(sl), None, stream))

    call()
    L.check_error(rt.infinirtStreamSynchronize(stream))
    eager = out.clone()
    assert_close(eager, oracle_of(oracle, inp), "eager")
    L.check_error(rt.infinirtStreamBeginCapture(stream, 0))
    call()
    L.check_error(rt.infinirtStreamEndCapture(stream, ctypes.byref(graph)))
    L.check_error(rt.infinirtGraphInstantiate(ctypes.byref(graph_exec), graph, None, None, 0))
    for replay in range(4):
        out.zero_()
        if replay != 2:
            ws.random_(0, 255)  # eager work between replays; the workspace content must not matter
        torch.cuda.synchronize()  # (replay 2 runs on what replay 1 left: cleared flags, first-tile entries that match)
        L.check_error(rt.infinirtGraphLuanch(graph_exec, stream))
        L.check_error(rt.infinirtStreamSynchronize(stream))
        assert torch.equal(out, eager), f"replay {replay}"
    L.check_error(rt.infinirtGraphExecDestroy(graph_exec))
    L.check_error(rt.infinirtGraphDestroy(graph))
    L.check_error(rt.infinirtStreamDestroy(stream))
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


def test_insufficient_workspace_is_refused_on_the_gpu_too(gpu_handle):
    inp = workloads.make_decode_inputs(custom("ws", torch.float16, 4, 8, 2, 128, 16, 1, 900, seed=61))
    q, k, v, bt, sl = to_device(inp)
    out = torch.full_like(q, 5.0)
    status, op = create_paged_attention(gpu_handle, out, q, k, v, bt, sl, None, inp.scale)
    size = workspace_size_attention(op)
    assert status == 0 and size > 0
    ws = torch.empty(size, dtype=torch.uint8, device=DEV)
    rc = L.LIBINFINIOP.infiniopPagedAttention(op, ptr(ws), size - 1, ptr(out), ptr(q), ptr(k), ptr(v), ptr(bt), ptr(sl), None, None)
    assert rc == L.InfiniStatus.INSUFFICIENT_WORKSPACE
    torch.cuda.synchronize()
    assert torch.all(out == 5)
    L.check_error(L.LIBINFINIOP.infiniopDestroyPagedAttentionDescriptor(op))


# ---- size-independent properties at full benchmark size ------------------------------------------------

def test_full_size_invariance_under_page_relocation(gpu_handle):
    """c2 at full size: moving every page to a new place in a bigger pool (and rewriting the table)
    changes no output bit that matters - checked to the tolerance, device against device."""
    inp = workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c2_llama3_8b_b32"])
    q, k, v, bt, sl = to_device(inp)
    base = run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale)
    nb = k.shape[0]
    perm = torch.randperm(nb, device=DEV, generator=torch.Generator(device=DEV).manual_seed(1))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nb, device=DEV)
    moved = run_paged_attention(gpu_handle, q, k[perm], v[perm], inv[bt], sl, inp.scale)
    assert_close(moved, base, "relocation")


def test_full_size_gqa_equals_mha_on_repeated_heads(gpu_handle):
    """c2 lengths, GQA 32/8 against MHA 32/32 on repeat_interleave'd pools (reduced batch to fit)."""
    cfg = custom("gqa_mha", torch.bfloat16, 8, 32, 8, 128, 16, 512, 4096, seed=67)
    inp = workloads.make_decode_inputs(cfg)
    q, k, v, bt, sl = to_device(inp)
    gqa = run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale)
    mha = run_paged_attention(gpu_handle, q, k.repeat_interleave(4, dim=1), v.repeat_interleave(4, dim=1), bt, sl, inp.scale)
    assert_close(mha, gqa, "gqa vs mha")


def test_full_size_linearity_in_v(gpu_handle):
    """Attention is linear in V: out(V1 + V2) = out(V1) + out(V2) for the same Q, K (c2 lengths)."""
    cfg = custom("linear", torch.float16, 8, 32, 8, 128, 16, 512, 4096, seed=71)
    inp = workloads.make_decode_inputs(cfg)
    q, k, v, bt, sl = to_device(inp)
    v2 = torch.randn_like(v, dtype=torch.float32).to(v.dtype) * 0.5
    a = run_paged_attention(gpu_handle, q, k, v, bt, sl, inp.scale).float()
    b = run_paged_attention(gpu_handle, q, k, v2, bt, sl, inp.scale).float()
    ab = run_paged_attention(gpu_handle, q, k, (v.float() + v2.float()).to(v.dtype), bt, sl, inp.scale).float()
    assert torch.all((ab - (a + b)).abs() <= 2 * ATOL + RTOL * (a + b).abs())
