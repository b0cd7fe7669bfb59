"""Pins the CPU oracle (oracle/paged_oracle.c) without the reference: the reference ships neither a
CPU implementation nor golden vectors for paged_attention / paged_caching, so every function of the
oracle is checked against something the mathematics fixes - an independent float64 formulation,
torch's own scaled_dot_product_attention, closed forms, and invariants - chosen so that a dropped
term, a wrong head / page index, a transposed operand or a wrong rounding fails at least one test."""
import numpy as np
import pytest
import torch

from infinicore_amd import workloads

from exact import exact_paged_attention, gather_sequence, ulp

DTYPES = [torch.float16, torch.bfloat16]


def small(dtype, B=3, H=8, Hkv=2, D=128, bs=16, lo=1, hi=200, seed=1, **kw):
    cfg = workloads.DecodeConfig("small", dtype, B, H, Hkv, D, bs, lo, hi, seed=seed, **kw)
    return workloads.make_decode_inputs(cfg)


def run(oracle, inp, **kw):
    return oracle.paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale, **kw)


def assert_within_rounding(got: torch.Tensor, exact: np.ndarray, dtype, slack=1.0):
    """got is exact rounded to dtype, plus fp32 accumulation noise far below one ulp."""
    g = got.to(torch.float64).numpy()
    err = np.abs(g - exact)
    bound = slack * ulp(dtype, exact) + 2e-6
    assert np.all(err <= bound), f"max err {err.max():.3g}, largest allowed {bound.max():.3g}"


# ---- storage formats ------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype,code", [(torch.float16, 0), (torch.bfloat16, 1)])
def test_to_float_all_65536_patterns(oracle, dtype, code):
    lib = oracle.load()
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    want = bits.view(dtype).to(torch.float32).numpy()
    got = np.array([lib.oracle_to_float(int(b) & 0xFFFF, code) for b in bits.tolist()], dtype=np.float32)
    same = (got == want) | (np.isnan(got) & np.isnan(want))
    assert same.all()


@pytest.mark.parametrize("dtype,code", [(torch.float16, 0), (torch.bfloat16, 1)])
def test_from_float_is_round_to_nearest_even(oracle, dtype, code):
    lib = oracle.load()
    rng = np.random.default_rng(3)
    samples = np.concatenate([
        rng.standard_normal(20000).astype(np.float32) * np.float32(10.0) ** rng.integers(-8, 6, 20000).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 65504.0, 65519.9, 65520.0, 1e10, -1e10, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                  2.0 ** -14, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -8, 1.0 + 3 * 2.0 ** -8, np.inf, -np.inf],
                 dtype=np.float32),
    ])
    want = torch.from_numpy(samples).to(dtype).view(torch.int16).numpy().astype(np.int64) & 0xFFFF
    got = np.array([lib.oracle_from_float(float(x), code) for x in samples.tolist()], dtype=np.int64)
    assert (got == want).all()


# ---- attention: independent formulations -----------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,D", [(8, 8, 128), (8, 2, 128), (4, 1, 64), (6, 3, 192)])
def test_matches_float64_two_pass_softmax(oracle, dtype, H, Hkv, D):
    inp = small(dtype, H=H, Hkv=Hkv, D=D)
    exact = exact_paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale)
    assert_within_rounding(run(oracle, inp), exact, dtype)


def test_matches_float64_on_the_plumbing_config_and_its_committed_fixture(oracle):
    """Config c1 (fp16 MHA, B=4, lens 1..256). The expected values are also committed as a fixture
    produced by tests/golden/make_c1_fixture.py from the float64 formulation."""
    from pathlib import Path
    inp = workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c1_plumbing_mha"])
    exact = exact_paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale)
    fixture = np.load(Path(__file__).parent / "golden" / "c1_plumbing_mha_expected_f64.npy")
    assert np.array_equal(fixture, exact)
    assert_within_rounding(run(oracle, inp), exact, torch.float16)


@pytest.mark.parametrize("dtype", DTYPES)
def test_matches_torch_sdpa_on_the_gathered_sequence(oracle, dtype):
    """After gathering, paged decode IS scaled_dot_product_attention with one query row (fp32 here)."""
    inp = small(dtype, B=2, H=8, Hkv=4, hi=150)
    got = run(oracle, inp).float()
    for s in range(2):
        L = int(inp.seq_lens[s])
        K = torch.from_numpy(gather_sequence(inp.k_cache, inp.block_tables[s], L)).float().permute(1, 0, 2)  # [Hkv, L, D]
        V = torch.from_numpy(gather_sequence(inp.v_cache, inp.block_tables[s], L)).float().permute(1, 0, 2)
        want = torch.nn.functional.scaled_dot_product_attention(
            inp.q[s].float().unsqueeze(1).unsqueeze(0), K.unsqueeze(0), V.unsqueeze(0), scale=inp.scale, enable_gqa=True)
        want = want[0, :, 0, :]
        assert torch.allclose(got[s], want, atol=float(ulp(dtype, np.array(4.0))), rtol=2.0 ** -7)


@pytest.mark.parametrize("dtype", DTYPES)
def test_alibi_matches_float64_with_bias(oracle, dtype):
    inp = small(dtype, B=2, H=8, Hkv=8, hi=120, seed=9)
    slopes = torch.tensor([2.0 ** -(i + 1) for i in range(8)], dtype=torch.float32)
    exact = exact_paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale, slopes.numpy())
    got = run(oracle, inp, alibi_slopes=slopes)
    assert_within_rounding(got, exact, dtype)
    # and the bias really matters: without it the answer differs
    assert not torch.equal(got, run(oracle, inp))


# ---- attention: closed forms -----------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_length_one_returns_the_value_row(oracle, dtype):
    inp = small(dtype, B=4, lo=1, hi=1)
    got = run(oracle, inp)
    for s in range(4):
        page = int(inp.block_tables[s, 0])
        want = inp.v_cache[page, :, 0, :].repeat_interleave(4, dim=0)  # H=8, Hkv=2
        assert torch.equal(got[s], want)  # v / (1 + 1e-6) rounds back to v


@pytest.mark.parametrize("dtype", DTYPES)
def test_equal_value_rows_are_returned_whatever_the_keys(oracle, dtype):
    inp = small(dtype, B=2, hi=90)
    row = torch.linspace(-2, 2, 128).to(dtype)
    inp.v_cache[:] = row
    got = run(oracle, inp)
    assert torch.allclose(got.float(), row.float().expand_as(got), atol=0, rtol=2.0 ** -7)


@pytest.mark.parametrize("dtype", DTYPES)
def test_zero_query_gives_the_mean_of_the_values(oracle, dtype):
    inp = small(dtype, B=2, H=4, Hkv=4, hi=60)
    inp.q.zero_()
    got = run(oracle, inp).double().numpy()
    for s in range(2):
        L = int(inp.seq_lens[s])
        V = gather_sequence(inp.v_cache, inp.block_tables[s], L)  # [L, Hkv, D]
        want = V.mean(axis=0)
        assert np.all(np.abs(got[s] - want) <= ulp(dtype, want) + 1e-6)


@pytest.mark.parametrize("dtype", DTYPES)
def test_one_dominant_key_selects_its_value_row(oracle, dtype):
    inp = small(dtype, B=1, H=4, Hkv=4, D=128, lo=100, hi=100, seed=4)
    L, hot = 100, 37
    page, row = int(inp.block_tables[0, hot // 16]), hot % 16
    inp.k_cache[page, :, row, :] = (inp.q[0] * 40).to(dtype)  # logit ~ 40*|q|^2*scale >> the others
    got = run(oracle, inp)
    assert torch.allclose(got[0].float(), inp.v_cache[page, :, row, :].float(), atol=1e-3, rtol=2.0 ** -7)


# ---- attention: invariants -------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_invariant_under_page_permutation(oracle, dtype):
    inp = small(dtype)
    base = run(oracle, inp)
    perm = torch.from_numpy(np.random.default_rng(5).permutation(inp.k_cache.shape[0]))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(len(perm))
    k2, v2 = inp.k_cache[perm], inp.v_cache[perm]  # new page i holds old page perm[i]
    moved = oracle.paged_attention(inp.q, k2, v2, inv[inp.block_tables], inp.seq_lens, inp.scale)
    assert torch.equal(base, moved)


@pytest.mark.parametrize("dtype", DTYPES)
def test_gqa_equals_mha_on_repeated_kv_heads(oracle, dtype):
    inp = small(dtype, H=8, Hkv=2)
    gqa = run(oracle, inp)
    k_rep = inp.k_cache.repeat_interleave(4, dim=1)
    v_rep = inp.v_cache.repeat_interleave(4, dim=1)
    mha = oracle.paged_attention(inp.q, k_rep, v_rep, inp.block_tables, inp.seq_lens, inp.scale)
    assert torch.equal(gqa, mha)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("splits", [1, 2, 4, 8])
def test_split_kv_formulation_agrees(oracle, dtype, splits):
    """Shards + combine (kernel_v2.cuh:340-616) against the single pass, including empty shards
    (sequences shorter than the number of splits)."""
    inp = small(dtype, B=5, lo=1, hi=70, seed=2)
    inp.seq_lens[0] = 1
    inp.seq_lens[1] = 3
    single = run(oracle, inp).double().numpy()
    split = run(oracle, inp, num_splits=splits).double().numpy()
    assert np.all(np.abs(single - split) <= ulp(dtype, single) + 1e-6)
    if splits == 1:
        assert np.array_equal(single, split)


@pytest.mark.parametrize("dtype", DTYPES)
def test_nothing_outside_the_sequence_is_read(oracle, dtype):
    inp = small(dtype, B=3, lo=5, hi=70, seed=6)
    base = run(oracle, inp)
    bs = 16
    k2, v2, bt = inp.k_cache.clone(), inp.v_cache.clone(), inp.block_tables.clone()
    for s in range(3):
        L = int(inp.seq_lens[s])
        last = (L - 1) // bs
        if L % bs:
            page = int(bt[s, last])
            k2[page, :, L % bs:, :] = float("nan")  # rows past the end of the sequence
            v2[page, :, L % bs:, :] = float("nan")
        bt[s, last + 1:] = 10 ** 9  # table entries past the last needed page
    assert torch.equal(base, oracle.paged_attention(inp.q, k2, v2, bt, inp.seq_lens, inp.scale))


def test_empty_sequences_leave_the_output_untouched(oracle):
    inp = small(torch.float16, B=4, seed=8)
    inp.seq_lens[1] = 0
    inp.seq_lens[3] = -5
    out = torch.full((4, 8, 128), 7.0, dtype=torch.float16)
    run(oracle, inp, out=out)
    assert torch.all(out[1] == 7) and torch.all(out[3] == 7)
    assert not torch.any(out[0] == 7) and not torch.any(out[2] == 7)


@pytest.mark.parametrize("dtype", DTYPES)
def test_strided_operands(oracle, dtype):
    """Pool stored [pages, rows, heads, d] and passed as a permuted view; q / out with padded rows."""
    inp = small(dtype, B=2, H=8, Hkv=4, hi=60)
    base = run(oracle, inp)
    k_perm = inp.k_cache.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    v_perm = inp.v_cache.permute(0, 2, 1, 3).contiguous().permute(0, 2, 1, 3)
    q_pad = torch.zeros(2, 8, 160, dtype=dtype)[:, :, :128]
    q_pad.copy_(inp.q)
    out_pad = torch.zeros(2, 10, 128, dtype=dtype)[:, :8, :]
    assert not k_perm.is_contiguous() and not q_pad.is_contiguous()
    got = oracle.paged_attention(q_pad, k_perm, v_perm, inp.block_tables, inp.seq_lens, inp.scale, out=out_pad)
    assert torch.equal(base, got)


# ---- the reference test's torch formulation ---------------------------------------------------------

@pytest.mark.parametrize("dtype", DTYPES)
def test_torch_formulations_agree_with_the_oracle_within_task_tolerance(oracle, dtype):
    """test/infiniop/paged_attention.py:38-88 restated (loop and vectorised) vs the kernel arithmetic:
    they differ in where they round (logits and probabilities in the storage dtype), which the
    tolerance atol 1e-2 / rtol 2e-3 covers."""
    inp = small(dtype, B=3, H=8, Hkv=2, hi=120)
    want = run(oracle, inp).float()
    loop = oracle.torch_reference_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale,
                                            vectorised=False).float()
    vec = oracle.torch_reference_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale).float()
    assert torch.equal(loop, vec)
    assert torch.all((loop - want).abs() <= 1e-2 + 2e-3 * want.abs())


# ---- paged_caching -----------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("permuted", [False, True])
def test_caching_is_a_byte_exact_scatter(oracle, dtype, permuted):
    rng = np.random.default_rng(11)
    ntok, Hkv, D, Dv, bs, NB = 50, 3, 64, 32, 8, 16
    k = torch.from_numpy(rng.standard_normal((ntok, Hkv, D), dtype=np.float32)).to(dtype)
    v = torch.from_numpy(rng.standard_normal((ntok, Hkv, Dv), dtype=np.float32)).to(dtype)
    slots = torch.from_numpy(rng.permutation(NB * bs)[:ntok].astype(np.int64))
    slots[::7] = -1
    if permuted:  # stored [pages, rows, heads, d], seen as [pages, heads, rows, d]
        k_cache = torch.full((NB, bs, Hkv, D), -777.0, dtype=dtype).permute(0, 2, 1, 3)
        v_cache = torch.full((NB, bs, Hkv, Dv), 555.0, dtype=dtype).permute(0, 2, 1, 3)
    else:
        k_cache = torch.full((NB, Hkv, bs, D), -777.0, dtype=dtype)
        v_cache = torch.full((NB, Hkv, bs, Dv), 555.0, dtype=dtype)
    # model: numpy fancy assignment on a copy
    k_want, v_want = k_cache.clone(), v_cache.clone()
    valid = slots >= 0
    k_want[slots[valid] // bs, :, slots[valid] % bs, :] = k[valid]
    v_want[slots[valid] // bs, :, slots[valid] % bs, :] = v[valid]
    oracle.paged_caching(k_cache, v_cache, k, v, slots)
    as_int = torch.int16 if dtype != torch.float32 else torch.int32
    assert torch.equal(k_cache.contiguous().view(as_int), k_want.contiguous().view(as_int))
    assert torch.equal(v_cache.contiguous().view(as_int), v_want.contiguous().view(as_int))
    # untouched slots still hold the sentinel; padding tokens went nowhere
    touched = int(valid.sum()) * Hkv * D
    assert int((k_cache != -777.0).sum()) <= touched
    # and the torch statement of the reference test gives the same pools
    k_ref, v_ref = oracle.torch_reference_caching(torch.full_like(k_want, -777.0), torch.full_like(v_want, 555.0), k, v, slots)
    assert torch.equal(k_ref, k_want) and torch.equal(v_ref, v_want)


def test_algorithmic_byte_counts():
    """The roofline's byte count, on a case small enough to count by hand."""
    cfg = workloads.DecodeConfig("t", torch.bfloat16, 2, 8, 2, 128, 16, 1, 64)
    lens = np.array([17, 32])
    kv = (17 + 32) * 2 * (128 + 128) * 2
    qo = 2 * 2 * 8 * 128 * 2
    idx = (2 + 2) * 8 + 2 * 8
    assert workloads.decode_algorithmic_bytes(cfg, lens) == kv + qo + idx
