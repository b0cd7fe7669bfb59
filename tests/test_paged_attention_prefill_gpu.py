"""GPU parity of infiniopPagedAttentionPrefill (through the C ABI) against the CPU oracle.

Tolerance: the one fixed for fp16 / bf16 attention output of the decode operator, atol 1e-2 and
rtol 2e-3 (tighter than the reference's own prefill test, which allows 1e-2/1e-2 for fp16 and
2e-2/2e-2 for bf16, test/infiniop/paged_attention_prefill.py:52-55).
"""
import os

import numpy as np
import pytest
import torch

from infinicore_amd import workloads

from capi import run_paged_attention_prefill
from test_paged_attention_gpu import DEV, ORACLE_THREADS, assert_close, climbing_keys

pytestmark = pytest.mark.gpu

SENTINEL = 7.0


def prefill_config(name, dtype, B, H, Hkv, D, bs, new, history, seed):
    return workloads.PrefillConfig(name, dtype, B, H, Hkv, D, bs, new[0], new[1], history[0], history[1], seed=seed)


def run_case(gpu_handle, oracle, inp, alibi=None, rows=None, index_dtype=torch.int64, what=None):
    """Runs the operator on the device and compares with the oracle: all rows, or the listed sample."""
    cfg = inp.config
    what = what or cfg.name
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache)]
    idx = [t.to(index_dtype).to(DEV) for t in (inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    alibi_dev = alibi.to(DEV) if alibi is not None else None
    print(f"case {what} T={inp.q.shape[0]} B={cfg.num_seqs} H={cfg.num_heads} Hkv={cfg.num_kv_heads} "
          f"D={inp.q.shape[2]} bs={cfg.block_size} dtype={cfg.dtype} idx={index_dtype} "
          f"kv[:4]={inp.seq_lens[:4].tolist()} cum[:5]={inp.cum_seq_lens_q[:5].tolist()}", flush=True)
    out = torch.full((*inp.q.shape[:-1], inp.v_cache.shape[-1]), SENTINEL, dtype=cfg.dtype, device=DEV)
    got = run_paged_attention_prefill(gpu_handle, *dev, *idx, inp.scale, alibi=alibi_dev, out=out).cpu()
    want, want_f32 = oracle.paged_attention_prefill(
        inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q, inp.scale,
        alibi_slopes=alibi, rows=rows, num_threads=ORACLE_THREADS, return_fp32=True,
        out=torch.full(got.shape, SENTINEL, dtype=cfg.dtype))
    if rows is not None:
        sel = torch.as_tensor(rows, dtype=torch.int64)
        assert_close(got[sel], want[sel], what, want_f32[sel])
    else:
        assert_close(got, want, what, want_f32)
    return got, want


# ---- the prefill configurations -----------------------------------------------------------------------

def test_p1_plumbing_mha(gpu_handle, oracle):
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(workloads.PREFILL_CONFIGS["p1_plumbing_mha"]))


def sample_rows(inp, per_seq=6, seed=0):
    """First, last and a few random rows of every sequence."""
    rng = np.random.default_rng(seed)
    cum = inp.cum_seq_lens_q.tolist()
    rows = []
    for s in range(len(cum) - 1):
        n = cum[s + 1] - cum[s]
        if n <= 0:
            continue
        picks = {0, n - 1, n // 2} | set(rng.integers(0, n, per_seq).tolist())
        rows += [cum[s] + j for j in sorted(picks)]
    return rows


def test_p2_llama3_8b_prompt_full_size_sampled_rows(gpu_handle, oracle):
    inp = workloads.make_prefill_inputs(workloads.PREFILL_CONFIGS["p2_llama3_8b_prompt"])
    run_case(gpu_handle, oracle, inp, rows=sample_rows(inp))


def test_p3_llama3_8b_chunked_full_size_sampled_rows(gpu_handle, oracle):
    inp = workloads.make_prefill_inputs(workloads.PREFILL_CONFIGS["p3_llama3_8b_chunked"])
    run_case(gpu_handle, oracle, inp, rows=sample_rows(inp, per_seq=3))


# ---- the reference's own test list ---------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize(
    "B,H,Hkv,D,bs,max_step,rounds,idx",
    [
        # test/infiniop/paged_attention_prefill.py:25-43 (I32 and I64 variants of each shape)
        (1, 1, 1, 128, 8, 16, 1, torch.int32),
        (1, 4, 4, 128, 8, 16, 4, torch.int64),
        (2, 8, 8, 128, 16, 32, 2, torch.int32),
        (4, 16, 16, 128, 8, 64, 3, torch.int64),
        (8, 64, 64, 128, 8, 16, 5, torch.int32),
        (16, 128, 128, 128, 8, 16, 4, torch.int64),
    ],
)
def test_reference_test_shapes_multi_round(gpu_handle, oracle, dtype, B, H, Hkv, D, bs, max_step, rounds, idx):
    """The reference test appends `rounds` batches of new tokens to every sequence and checks the last;
    here the last round is run: history = what the earlier rounds appended."""
    rng = np.random.default_rng(B * 131 + H + rounds)
    history_hi = max_step * (rounds - 1)
    history_lo = rounds - 1  # at least one token per earlier round
    cfg = prefill_config("reference_shape", dtype, B, H, Hkv, D, bs, (1, max_step), (history_lo, history_hi),
                         seed=int(rng.integers(1 << 30)))
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg), index_dtype=idx)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("idx", [torch.int32, torch.int64])
def test_reference_mla_shape(gpu_handle, oracle, dtype, idx):
    """(2, 16, 1, 576, 16, 8, 2, idx, 512): DeepSeek MLA, value size 512 (paged_attention_prefill.py:41-42)."""
    cfg = prefill_config("mla", dtype, 2, 16, 1, 576, 16, (1, 8), (1, 8), seed=77)
    inp = workloads.make_prefill_inputs(cfg)
    inp.v_cache = inp.v_cache[..., :512].contiguous()
    run_case(gpu_handle, oracle, inp, index_dtype=idx)


def mla_inputs(name, dtype, B, H, bs, new, history, seed):
    """Latent-attention caches: keys of 576 elements, values of 512, one KV head."""
    inp = workloads.make_prefill_inputs(prefill_config(name, dtype, B, H, 1, 576, bs, new, history, seed=seed))
    inp.v_cache = inp.v_cache[..., :512].contiguous()
    return inp


@pytest.mark.parametrize("kernel", ["tiled", "generic"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H", [16, 128, 5])
def test_mla_ragged_batches(gpu_handle, oracle, monkeypatch, H, dtype, kernel):
    """Keys 576 / values 512 on the matrix-core kernel (64 rows per workgroup, 32-token steps) and on the
    element-wise one: 16 heads (a tensor-parallel shard), all 128, and a head count that fills no tile."""
    if kernel == "generic":
        monkeypatch.setenv("INFINIOP_AMD_PREFILL_KERNEL", "generic")
    small = kernel == "generic" or H == 128
    inp = mla_inputs(f"mla_h{H}_{kernel}", dtype, 3, H, 16, (1, 30 if small else 200), (0, 80 if small else 500), seed=500 + H)
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("bs", [8, 64])
def test_mla_page_sizes_alibi_and_int32(gpu_handle, oracle, bs):
    inp = mla_inputs(f"mla_bs{bs}", torch.bfloat16, 3, 16, bs, (1, 120), (0, 300), seed=520 + bs)
    slopes = torch.tensor([2.0 ** -(i % 5 + 1) for i in range(16)], dtype=torch.float32)
    run_case(gpu_handle, oracle, inp, alibi=slopes, index_dtype=torch.int32)


@pytest.mark.parametrize("kernel", ["tiled", "generic"])
def test_mla_values_as_a_view_of_the_keys(gpu_handle, oracle, monkeypatch, kernel):
    """The latent layout of DeepSeek-style caches: one tensor of 576 columns per token, the values being its first
    512 columns (a V row stride of 576 elements)."""
    if kernel == "generic":
        monkeypatch.setenv("INFINIOP_AMD_PREFILL_KERNEL", "generic")
    inp = mla_inputs(f"mla_view_{kernel}", torch.bfloat16, 3, 16, 16, (1, 40), (0, 150), seed=560)
    k_dev = inp.k_cache.to(DEV)
    v_dev = k_dev[..., :512]
    idx = [t.to(DEV) for t in (inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    got = run_paged_attention_prefill(gpu_handle, inp.q.to(DEV), k_dev, v_dev, *idx, inp.scale).cpu()
    want, want_f32 = oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.k_cache[..., :512], inp.block_tables, inp.seq_lens,
                                                    inp.cum_seq_lens_q, inp.scale, num_threads=ORACLE_THREADS, return_fp32=True)
    assert_close(got, want, f"mla_view_{kernel}", want_f32)


def test_mla_column_layout_and_garbage(gpu_handle, oracle):
    """V with a distinct constant per column makes the expected output that constant (every one of the 512 output
    columns lands where it belongs); NaN beyond the sequences must not leak in."""
    inp = mla_inputs("mla_cols", torch.float16, 3, 16, 16, (5, 90), (3, 200), seed=540)
    cfg = inp.config
    ramp = ((torch.arange(512, dtype=torch.float32) - 256) / 16).to(torch.float16)
    inp.v_cache[:] = ramp
    for s in range(cfg.num_seqs):
        L = int(inp.seq_lens[s])
        if L % 16:
            page = int(inp.block_tables[s, (L - 1) // 16])
            inp.k_cache[page, :, L % 16:, :] = float("nan")
            inp.v_cache[page, :, L % 16:, :] = float("nan")
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    got = run_paged_attention_prefill(gpu_handle, *dev, inp.scale).float().cpu()
    want = ramp.float().expand_as(got)
    assert torch.allclose(got, want, atol=2e-3 * float(ramp.float().abs().max()), rtol=0), (got - want).abs().max()


# ---- heads of 576 with values of 576 (the decode test list of the reference has the shape,
# test/infiniop/paged_attention.py:106): the matrix-core kernel of the latent shape with 36 value blocks -------------

@pytest.mark.parametrize("kernel", ["tiled", "generic"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("H,Hkv", [(16, 16), (20, 1), (8, 2)])
def test_head_576_with_values_of_576(gpu_handle, oracle, monkeypatch, dtype, H, Hkv, kernel):
    if kernel == "generic":
        monkeypatch.setenv("INFINIOP_AMD_PREFILL_KERNEL", "generic")
    small = kernel == "generic"
    cfg = prefill_config(f"h576_{H}_{Hkv}_{kernel}", dtype, 3, H, Hkv, 576, 16, (1, 30 if small else 150), (0, 80 if small else 400), seed=600 + H)
    got, _ = run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg))
    assert got.shape[-1] == 576


def test_head_576_column_layout_garbage_alibi_and_int32(gpu_handle, oracle):
    """Every one of the 576 output columns lands where it belongs (V with a distinct constant per column), NaN beyond the
    sequences does not leak in; then the same inputs with random values, ALiBi and 32-bit indices against the oracle."""
    inp = workloads.make_prefill_inputs(prefill_config("h576_cols", torch.float16, 3, 8, 2, 576, 16, (5, 90), (3, 200), seed=640))
    values = inp.v_cache.clone()
    ramp = ((torch.arange(576, dtype=torch.float32) - 288) / 16).to(torch.float16)
    inp.v_cache[:] = ramp
    for s in range(inp.config.num_seqs):
        L = int(inp.seq_lens[s])
        if L % 16:
            page = int(inp.block_tables[s, (L - 1) // 16])
            inp.k_cache[page, :, L % 16:, :] = float("nan")
            inp.v_cache[page, :, L % 16:, :] = float("nan")
            values[page, :, L % 16:, :] = float("nan")
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    got = run_paged_attention_prefill(gpu_handle, *dev, inp.scale).float().cpu()
    want = ramp.float().expand_as(got)
    assert torch.allclose(got, want, atol=2e-3 * float(ramp.float().abs().max()), rtol=0), (got - want).abs().max()
    inp.v_cache = values
    slopes = torch.tensor([2.0 ** -(i % 5 + 1) for i in range(8)], dtype=torch.float32)
    run_case(gpu_handle, oracle, inp, alibi=slopes, index_dtype=torch.int32)


# ---- kernel variants --------------------------------------------------------------------------------------

@pytest.mark.parametrize("groups", ["1", "2"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_every_row_block_size_of_the_tiled_kernel(gpu_handle, oracle, monkeypatch, groups, dtype):
    monkeypatch.setenv("INFINIOP_AMD_PREFILL_GROUPS", groups)
    cfg = prefill_config(f"groups{groups}", dtype, 5, 16, 4, 128, 16, (1, 300), (0, 500), seed=31)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg))


@pytest.mark.parametrize("groups", ["1", "2"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_scores_that_climb_along_the_sequence(gpu_handle, oracle, monkeypatch, groups, dtype):
    """Every row's running maximum moves in every step, mostly by less than the rescaling threshold and
    at the jumps by much more (the keys are laid out by test_paged_attention_gpu.climbing_keys)."""
    monkeypatch.setenv("INFINIOP_AMD_PREFILL_GROUPS", groups)
    cfg = prefill_config(f"climb{groups}", dtype, 3, 16, 4, 128, 16, (100, 400), (0, 700), seed=73)
    inp = workloads.make_prefill_inputs(cfg)
    q = inp.q.clone()
    climbing_keys(inp, step_log2=0.05, jump_every=150, jump_log2=12.0)
    # keep distinct queries per token (same direction, different lengths), so rows differ
    scale_rows = torch.linspace(0.5, 1.5, q.shape[0])[:, None, None]
    inp.q[:] = (inp.q.float() * scale_rows).to(cfg.dtype)
    run_case(gpu_handle, oracle, inp)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_element_wise_kernel_on_a_tiled_shape(gpu_handle, oracle, monkeypatch, dtype):
    monkeypatch.setenv("INFINIOP_AMD_PREFILL_KERNEL", "generic")
    cfg = prefill_config("generic", dtype, 3, 8, 2, 128, 16, (1, 40), (0, 100), seed=37)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg))


@pytest.mark.parametrize("kernel", ["tiled-1", "tiled-2", "generic"])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("D", [64, 192, 256])
def test_other_head_sizes(gpu_handle, oracle, monkeypatch, D, dtype, kernel):
    """Head sizes 64 / 192 / 256 on the matrix-core kernel, 64 and 128 rows per workgroup (head 192 takes steps of 32
    tokens with 64 rows and of 64 tokens with 128), and on the element-wise one."""
    if kernel == "generic":
        monkeypatch.setenv("INFINIOP_AMD_PREFILL_KERNEL", "generic")
    else:
        monkeypatch.setenv("INFINIOP_AMD_PREFILL_GROUPS", kernel[-1])
    small = kernel == "generic"
    cfg = prefill_config(f"head{D}_{kernel}", dtype, 4, 8, 4, D, 16, (1, 40 if small else 260), (0, 100 if small else 400),
                         seed=41 + D)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg))


@pytest.mark.parametrize("D,groups", [(64, "1"), (64, "2"), (192, "1"), (192, "2"), (256, "1"), (256, "2")])
def test_other_head_sizes_pages_of_8_alibi_and_int32(gpu_handle, oracle, monkeypatch, D, groups):
    monkeypatch.setenv("INFINIOP_AMD_PREFILL_GROUPS", groups)
    cfg = prefill_config(f"mix{D}", torch.bfloat16, 3, 12, 2, D, 8, (1, 150), (0, 300), seed=91 + D)
    slopes = torch.tensor([2.0 ** -(i % 6 + 1) for i in range(12)], dtype=torch.float32)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg), alibi=slopes, index_dtype=torch.int32)


@pytest.mark.parametrize("groups", ["1", "2"])
@pytest.mark.parametrize("D", [64, 192, 256])
def test_other_head_sizes_column_layout_and_garbage(gpu_handle, oracle, monkeypatch, D, groups):
    """V with a distinct constant per column makes the expected output that constant (every output column
    lands where it belongs); NaN beyond the sequences must not leak in."""
    monkeypatch.setenv("INFINIOP_AMD_PREFILL_GROUPS", groups)
    cfg = prefill_config(f"cols{D}", torch.float16, 3, 8, 2, D, 16, (5, 90), (3, 200), seed=97 + D)
    inp = workloads.make_prefill_inputs(cfg)
    ramp = ((torch.arange(D, dtype=torch.float32) - D / 2) / 8).to(torch.float16)
    inp.v_cache[:] = ramp
    for s in range(cfg.num_seqs):
        L = int(inp.seq_lens[s])
        if L % 16:
            page = int(inp.block_tables[s, (L - 1) // 16])
            inp.k_cache[page, :, L % 16:, :] = float("nan")
            inp.v_cache[page, :, L % 16:, :] = float("nan")
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    got = run_paged_attention_prefill(gpu_handle, *dev, inp.scale).float().cpu()
    want = ramp.float().expand_as(got)
    assert torch.allclose(got, want, atol=2e-3 * float(ramp.float().abs().max()), rtol=0), (got - want).abs().max()


@pytest.mark.parametrize("bs", [4, 8, 32, 128, 24])
def test_page_sizes(gpu_handle, oracle, bs):
    """Powers of two from 8 run the tiled kernel (8 = two pages per 16-token tile), the others the element-wise one."""
    cfg = prefill_config(f"page{bs}", torch.bfloat16, 4, 8, 2, 128, bs, (1, 150), (0, 300), seed=43 + bs)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg))


@pytest.mark.parametrize("idx", [torch.int32, torch.uint32, torch.int64])
def test_index_dtypes(gpu_handle, oracle, idx):
    cfg = prefill_config("index", torch.float16, 3, 8, 8, 128, 16, (1, 70), (0, 90), seed=47)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg), index_dtype=idx)


@pytest.mark.parametrize("H,Hkv", [(32, 8), (8, 1), (6, 2), (40, 40), (24, 8)])
def test_group_sizes(gpu_handle, oracle, H, Hkv):
    """Rows of a workgroup are (token, head-in-group) pairs: group sizes that do and do not divide 16."""
    cfg = prefill_config(f"gqa{H}_{Hkv}", torch.bfloat16, 3, H, Hkv, 128, 16, (1, 90), (0, 200), seed=53 + H)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kernel", ["tiled", "generic"])
def test_alibi(gpu_handle, oracle, monkeypatch, dtype, kernel):
    if kernel == "generic":
        monkeypatch.setenv("INFINIOP_AMD_PREFILL_KERNEL", "generic")
    cfg = prefill_config("alibi", dtype, 3, 8, 2, 128, 16, (1, 120), (0, 200), seed=59)
    slopes = torch.tensor([2.0 ** -(i / 2 + 1) for i in range(8)], dtype=torch.float32)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg), alibi=slopes)


@pytest.mark.parametrize("seed", range(int(os.environ.get("INFINICORE_AMD_TEST_SWEEP_SEEDS", "48"))))
def test_random_shapes_row_blocks_and_dtypes(gpu_handle, oracle, monkeypatch, seed):
    """Every knob drawn at random from one seed: head size (with keys of 576 and values of 512 or 576), group size,
    page size, batch, new-token and history ranges, dtype, index dtype, ALiBi and rows per workgroup."""
    rng = np.random.default_rng(2000 + seed)
    D, Dv = [(64, 64), (128, 128), (128, 128), (192, 192), (256, 256), (576, 512), (576, 576)][rng.integers(0, 7)]
    Hkv = int(rng.choice([1, 2, 4])) if D != 576 else int(rng.choice([1, 1, 2]))
    group = int(rng.choice([1, 2, 3, 4, 7])) if D != 576 else int(rng.choice([1, 5, 16, 20]))
    bs = int(rng.choice([8, 16, 16, 32, 64]))
    B = int(rng.choice([1, 3, 9])) if D != 576 else int(rng.choice([1, 3]))
    new = (1, int(rng.choice([1, 20, 150, 400]))) if D != 576 else (1, int(rng.choice([1, 20, 150])))
    history = (0, int(rng.choice([0, 50, 700]))) if D != 576 else (0, int(rng.choice([0, 50, 300])))
    dtype = [torch.float16, torch.bfloat16][rng.integers(0, 2)]
    idx = [torch.int64, torch.int32, torch.uint32][rng.integers(0, 3)]
    groups = ["1", "2"][rng.integers(0, 2)]
    use_alibi = bool(rng.integers(0, 2))
    monkeypatch.setenv("INFINIOP_AMD_PREFILL_GROUPS", groups)
    H = Hkv * group
    cfg = prefill_config(f"sweep{seed}", dtype, B, H, Hkv, D, bs, new, history, seed=800 + seed)
    slopes = torch.tensor(rng.uniform(0.001, 0.3, H), dtype=torch.float32) if use_alibi else None
    print(f"sweep {seed}: D={D}/{Dv} H={H}/{Hkv} bs={bs} B={B} new={new} history={history} {dtype} {idx} rows/wg={groups} "
          f"alibi={use_alibi}", flush=True)
    inp = workloads.make_prefill_inputs(cfg)
    if Dv != D:
        inp.v_cache = inp.v_cache[..., :Dv].contiguous()
    run_case(gpu_handle, oracle, inp, alibi=slopes, index_dtype=idx)


# ---- edge cases ---------------------------------------------------------------------------------------------

def test_one_new_token_per_sequence_equals_decode(gpu_handle, oracle):
    from capi import run_paged_attention
    cfg = prefill_config("decode_like", torch.bfloat16, 6, 32, 8, 128, 16, (1, 1), (0, 700), seed=61)
    inp = workloads.make_prefill_inputs(cfg)
    got, _ = run_case(gpu_handle, oracle, inp)
    dec = run_paged_attention(gpu_handle, inp.q.to(DEV), inp.k_cache.to(DEV), inp.v_cache.to(DEV),
                              inp.block_tables.to(DEV), inp.seq_lens.to(DEV), inp.scale).cpu()
    assert_close(got, dec, "prefill of one token vs decode",
                 oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                        return_fp32=True)[1])


@pytest.mark.parametrize("kernel", ["tiled", "generic"])
def test_rows_nobody_owns_negative_history_and_empty_sequences_stay_untouched(gpu_handle, oracle, monkeypatch, kernel):
    if kernel == "generic":
        monkeypatch.setenv("INFINIOP_AMD_PREFILL_KERNEL", "generic")
    cfg = prefill_config("edges", torch.float16, 4, 8, 2, 128, 16, (5, 60), (0, 80), seed=67)
    inp = workloads.make_prefill_inputs(cfg)
    cum = inp.cum_seq_lens_q.tolist()
    # three extra rows past cum[-1]; sequence 1 shorter than its new tokens (its first rows see nothing);
    # an empty sequence inserted between 2 and 3
    inp.q = torch.cat([inp.q, torch.randn(3, 8, 128).half()])
    new1 = cum[2] - cum[1]
    inp.seq_lens = inp.seq_lens.clone()
    inp.seq_lens[1] = new1 - 4
    inp.seq_lens = torch.cat([inp.seq_lens[:3], torch.tensor([9]), inp.seq_lens[3:]])
    inp.cum_seq_lens_q = torch.tensor(cum[:4] + [cum[3]] + cum[4:])
    inp.block_tables = torch.cat([inp.block_tables[:3], inp.block_tables[:1], inp.block_tables[3:]])
    got, want = run_case(gpu_handle, oracle, inp)
    T = cum[-1]
    assert (got[T:] == SENTINEL).all() and (want[T:] == SENTINEL).all()
    assert (got[cum[1]:cum[1] + 4] == SENTINEL).all()
    assert not (got[cum[1] + 4] == SENTINEL).all()


def test_garbage_beyond_the_sequences_is_never_used(gpu_handle, oracle):
    """NaN in every cache row past each sequence's length and huge ids in unused table entries."""
    cfg = prefill_config("poison", torch.bfloat16, 4, 8, 2, 128, 16, (3, 100), (0, 150), seed=71)
    inp = workloads.make_prefill_inputs(cfg)
    bs = cfg.block_size
    for s in range(cfg.num_seqs):
        L = int(inp.seq_lens[s])
        nb = (L + bs - 1) // bs
        if L % bs:
            page = int(inp.block_tables[s, nb - 1])
            inp.k_cache[page, :, L % bs:, :] = float("nan")
            inp.v_cache[page, :, L % bs:, :] = float("nan")
        inp.block_tables[s, nb:] = 1 << 40
    run_case(gpu_handle, oracle, inp)


def test_strided_operands(gpu_handle, oracle):
    """q / out rows with a gap, caches stored token-major ([blocks, page, heads, dim] permuted to the
    operator's [blocks, heads, page, dim] view), a block table wider than needed."""
    cfg = prefill_config("strided", torch.float16, 3, 8, 2, 128, 16, (1, 80), (0, 120), seed=73)
    inp = workloads.make_prefill_inputs(cfg)
    T = inp.q.shape[0]
    q_big = torch.zeros(T, 8, 256, dtype=torch.float16, device=DEV)
    q_big[..., :128] = inp.q.to(DEV)
    out_big = torch.full((T, 8, 256), SENTINEL, dtype=torch.float16, device=DEV)
    k_dev = inp.k_cache.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)
    v_dev = inp.v_cache.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)
    bt = torch.zeros(3, inp.block_tables.shape[1] + 5, dtype=torch.int64)
    bt[:, :inp.block_tables.shape[1]] = inp.block_tables
    got = run_paged_attention_prefill(gpu_handle, q_big[..., :128], k_dev, v_dev, bt.to(DEV)[:, :],
                                      inp.seq_lens.to(DEV), inp.cum_seq_lens_q.to(DEV), inp.scale,
                                      out=out_big[..., :128]).cpu()
    want, want_f32 = oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                                    inp.cum_seq_lens_q, inp.scale, return_fp32=True)
    assert_close(got, want, "strided", want_f32)
    assert (out_big[..., 128:] == SENTINEL).all()


def test_unaligned_base_addresses_take_the_element_wise_kernel(gpu_handle, oracle):
    cfg = prefill_config("unaligned", torch.bfloat16, 2, 8, 2, 128, 16, (1, 30), (0, 60), seed=79)
    inp = workloads.make_prefill_inputs(cfg)
    T = inp.q.shape[0]
    flat = torch.zeros(T * 8 * 128 + 1, dtype=torch.bfloat16, device=DEV)
    q_odd = flat[1:].view(T, 8, 128)
    q_odd.copy_(inp.q.to(DEV))
    got = run_paged_attention_prefill(gpu_handle, q_odd, inp.k_cache.to(DEV), inp.v_cache.to(DEV),
                                      inp.block_tables.to(DEV), inp.seq_lens.to(DEV), inp.cum_seq_lens_q.to(DEV),
                                      inp.scale).cpu()
    want, want_f32 = oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                                    inp.cum_seq_lens_q, inp.scale, return_fp32=True)
    assert_close(got, want, "unaligned", want_f32)


def test_many_short_sequences(gpu_handle, oracle):
    """More sequences than one wavefront scans at a time (the row-block lookup walks them 64 at a time)."""
    cfg = prefill_config("many", torch.float16, 150, 8, 8, 128, 16, (0, 9), (0, 40), seed=83)
    run_case(gpu_handle, oracle, workloads.make_prefill_inputs(cfg))


# ---- properties at full size -----------------------------------------------------------------------------

def test_p2_page_permutation_invariance_and_determinism(gpu_handle):
    """Moving every page to a different physical slot (table updated) must not change a single bit, and
    neither must running twice."""
    inp = workloads.make_prefill_inputs(workloads.PREFILL_CONFIGS["p2_llama3_8b_prompt"])
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    first = run_paged_attention_prefill(gpu_handle, *dev, inp.scale)
    again = run_paged_attention_prefill(gpu_handle, *dev, inp.scale)
    assert torch.equal(first, again)
    nb = inp.k_cache.shape[0]
    perm = torch.from_numpy(np.random.default_rng(5).permutation(nb))
    inverse = torch.empty_like(perm)
    inverse[perm] = torch.arange(nb)
    k2, v2 = inp.k_cache[perm].to(DEV), inp.v_cache[perm].to(DEV)  # new slot i holds old page perm[i]
    moved = run_paged_attention_prefill(gpu_handle, dev[0], k2, v2, inverse[inp.block_tables].to(DEV), dev[4], dev[5],
                                        inp.scale)
    assert torch.equal(first, moved)


def test_ops_front_end(oracle):
    from infinicore_amd import ops
    cfg = prefill_config("ops", torch.float16, 3, 8, 2, 128, 16, (1, 50), (0, 70), seed=89)
    inp = workloads.make_prefill_inputs(cfg)
    dev = [t.to(DEV) for t in (inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.cum_seq_lens_q)]
    got = ops.paged_attention_prefill(*dev, None, inp.scale)
    again = ops.paged_attention_prefill(*dev, scale=inp.scale)  # served from the descriptor cache
    want, want_f32 = oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                                    inp.cum_seq_lens_q, inp.scale, return_fp32=True)
    assert_close(got, want, "ops.paged_attention_prefill", want_f32)
    assert torch.equal(got, again)
