"""Pins the prefill function of the CPU oracle (oracle_paged_attention_prefill) without the
reference, which ships neither a CPU implementation nor golden vectors for paged_attention_prefill:
an independent float64 masked softmax on gathered K/V, torch's scaled_dot_product_attention with an
explicit causal mask, the identity "row j of a sequence == decode over its first history + j + 1
tokens" against the separately pinned decode oracle, and the edge cases of the row -> sequence
lookup. A wrong history offset, an off-by-one in the visible range, a wrong row -> sequence map or a
wrong ALiBi origin fails at least one of them."""
import numpy as np
import pytest
import torch

from infinicore_amd import workloads

from exact import gather_sequence, ulp

DTYPES = [torch.float16, torch.bfloat16]


def small(dtype, B=3, H=8, Hkv=2, D=128, bs=16, new=(1, 40), history=(0, 70), seed=1):
    cfg = workloads.PrefillConfig("small", dtype, B, H, Hkv, D, bs, new[0], new[1], history[0], history[1], seed=seed)
    return workloads.make_prefill_inputs(cfg)


def run(oracle, inp, **kw):
    return oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                          inp.cum_seq_lens_q, inp.scale, **kw)


def exact_prefill(inp, alibi_slopes=None) -> np.ndarray:
    """float64 [total_q, H, Dv] by the textbook two-pass softmax; rows that see nothing are NaN."""
    q = inp.q.to(torch.float64).numpy()
    T, H, _ = q.shape
    group = H // inp.k_cache.shape[1]
    out = np.full((T, H, inp.v_cache.shape[3]), np.nan)
    cum = inp.cum_seq_lens_q.tolist()
    for s in range(len(cum) - 1):
        total = int(inp.seq_lens[s])
        new = cum[s + 1] - cum[s]
        K = gather_sequence(inp.k_cache, inp.block_tables[s], max(total, 0))
        V = gather_sequence(inp.v_cache, inp.block_tables[s], max(total, 0))
        for j in range(new):
            n = total - new + j + 1
            if n <= 0:
                continue
            for h in range(H):
                logits = float(inp.scale) * (K[:n, h // group, :] @ q[cum[s] + j, h])
                if alibi_slopes is not None:
                    logits = logits + float(alibi_slopes[h]) * (np.arange(n) - (n - 1))
                p = np.exp(logits - logits.max())
                out[cum[s] + j, h] = (p / p.sum()) @ V[:n, h // group, :]
    return out


def assert_within_rounding(got, exact, dtype):
    g = got.to(torch.float64).numpy()
    seen = ~np.isnan(exact)
    err = np.abs(g - exact)[seen]
    bound = (ulp(dtype, exact) + 2e-6)[seen]
    assert np.all(err <= bound), f"max err {err.max():.3g}, largest allowed {bound.max():.3g}"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,Hkv,D,bs", [(8, 8, 128, 16), (8, 2, 128, 8), (4, 1, 64, 16), (6, 3, 192, 4)])
def test_matches_float64_masked_softmax(oracle, dtype, H, Hkv, D, bs):
    inp = small(dtype, H=H, Hkv=Hkv, D=D, bs=bs)
    assert_within_rounding(run(oracle, inp), exact_prefill(inp), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_matches_float64_with_alibi(oracle, dtype):
    inp = small(dtype, seed=5)
    slopes = torch.tensor([2.0 ** -(i + 1) for i in range(8)], dtype=torch.float32)
    assert_within_rounding(run(oracle, inp, alibi_slopes=slopes), exact_prefill(inp, slopes), dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_matches_torch_sdpa_with_causal_offset_mask(oracle, dtype):
    inp = small(dtype, H=8, Hkv=2, seed=9)
    got = run(oracle, inp).float()
    cum = inp.cum_seq_lens_q.tolist()
    for s in range(len(cum) - 1):
        total, new = int(inp.seq_lens[s]), cum[s + 1] - cum[s]
        K = torch.from_numpy(gather_sequence(inp.k_cache, inp.block_tables[s], total)).float()
        V = torch.from_numpy(gather_sequence(inp.v_cache, inp.block_tables[s], total)).float()
        Q = inp.q[cum[s]:cum[s + 1]].float()
        mask = torch.arange(total).view(1, -1) <= (total - new + torch.arange(new)).view(-1, 1)
        want = torch.nn.functional.scaled_dot_product_attention(
            Q.permute(1, 0, 2).unsqueeze(0), K.permute(1, 0, 2).unsqueeze(0), V.permute(1, 0, 2).unsqueeze(0),
            attn_mask=mask, scale=inp.scale, enable_gqa=True)[0].permute(1, 0, 2)
        tol = 2.0 ** (-10 if dtype == torch.float16 else -7)
        assert torch.allclose(got[cum[s]:cum[s + 1]], want, atol=tol * 1.01, rtol=tol * 1.01)


@pytest.mark.parametrize("dtype", DTYPES)
def test_every_row_equals_decode_over_its_visible_prefix(oracle, dtype):
    """Bit for bit: the prefill recurrence of one row is the decode recurrence over history + j + 1 tokens."""
    inp = small(dtype, B=4, H=4, Hkv=2, seed=11)
    slopes = torch.tensor([0.5, 0.25, 0.125, 0.0625])
    got = run(oracle, inp, alibi_slopes=slopes)
    cum = inp.cum_seq_lens_q.tolist()
    for s in range(len(cum) - 1):
        new = cum[s + 1] - cum[s]
        for j in range(new):
            n = int(inp.seq_lens[s]) - new + j + 1
            row = cum[s] + j
            want = oracle.paged_attention(inp.q[row:row + 1], inp.k_cache, inp.v_cache, inp.block_tables[s:s + 1],
                                          torch.tensor([n]), inp.scale, alibi_slopes=slopes)
            assert torch.equal(got[row], want[0]), (s, j)


def test_rows_without_a_sequence_or_without_visible_tokens_are_left_alone(oracle):
    inp = small(torch.float16, B=3, seed=13)
    T = inp.q.shape[0]
    # two extra query rows past cum[-1]; sequence 1 claims more new tokens than its K/V length
    q = torch.cat([inp.q, torch.randn(2, *inp.q.shape[1:]).half()])
    lens = inp.seq_lens.clone()
    cum = inp.cum_seq_lens_q
    new1 = int(cum[2] - cum[1])
    lens[1] = max(new1 - 3, 0)  # history = -3 (or less): the first rows of sequence 1 see nothing
    sentinel = torch.full((T + 2, inp.q.shape[1], inp.v_cache.shape[3]), 7.0, dtype=torch.float16)
    got = oracle.paged_attention_prefill(q, inp.k_cache, inp.v_cache, inp.block_tables, lens, cum, inp.scale,
                                         out=sentinel.clone())
    assert torch.equal(got[T:], sentinel[T:])
    blind = min(3, new1) if new1 >= 3 else new1
    assert torch.equal(got[int(cum[1]):int(cum[1]) + blind], sentinel[:blind])
    if new1 > 3:
        assert not torch.equal(got[int(cum[1]) + 3], sentinel[0])
    # the other sequences are unaffected by the change
    ref = run(oracle, inp)
    assert torch.equal(got[:int(cum[1])], ref[:int(cum[1])]) and torch.equal(got[int(cum[2]):T], ref[int(cum[2]):])


def test_empty_sequences_in_the_batch(oracle):
    """cum_seq_lens_q with repeated entries: a sequence with no new tokens owns no row."""
    inp = small(torch.bfloat16, B=2, seed=17)
    cum = inp.cum_seq_lens_q.tolist()
    cum5 = torch.tensor([0, 0, cum[1], cum[1], cum[2]])
    lens5 = torch.tensor([5, int(inp.seq_lens[0]), 0, int(inp.seq_lens[1])])
    tables5 = torch.stack([inp.block_tables[0], inp.block_tables[0], inp.block_tables[1], inp.block_tables[1]])
    got = oracle.paged_attention_prefill(inp.q, inp.k_cache, inp.v_cache, tables5, lens5, cum5, inp.scale)
    assert torch.equal(got, run(oracle, inp))


def test_row_subset_evaluates_only_those_rows(oracle):
    inp = small(torch.float16, seed=19)
    full, full32 = run(oracle, inp, return_fp32=True)
    rows = [0, 3, inp.q.shape[0] - 1]
    part, part32 = run(oracle, inp, rows=rows, return_fp32=True)
    for r in range(inp.q.shape[0]):
        if r in rows:
            assert torch.equal(part[r], full[r]) and torch.equal(part32[r], full32[r])
        else:
            assert torch.count_nonzero(part[r]) == 0 and torch.isnan(part32[r]).all()


@pytest.mark.parametrize("dtype", DTYPES)
def test_torch_statement_of_the_reference_test_agrees(oracle, dtype):
    """The torch function the reference's prefill test uses as its expected value (probabilities rounded
    to the storage dtype before P.V) agrees with the oracle within that test's tolerance
    (test/infiniop/paged_attention_prefill.py:52-55: fp16 1e-2/1e-2, bf16 2e-2/2e-2)."""
    inp = small(dtype, H=8, Hkv=8, seed=23)
    want = oracle.torch_reference_prefill(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens,
                                          inp.cum_seq_lens_q, inp.scale)
    tol = 1e-2 if dtype == torch.float16 else 2e-2
    assert torch.allclose(run(oracle, inp).float(), want.float(), atol=tol, rtol=tol)
