"""Host-side logic that needs no GPU: the benchmark's command line contract, the seeded workload generators
and their byte / flop accounting."""
import subprocess
import sys
from pathlib import Path

import numpy as np
import pytest
import torch

from infinicore_amd import workloads

ROOT = Path(__file__).resolve().parents[1]


def test_bench_refuses_more_than_one_gpu():
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert proc.returncode == 2
    assert "ONE GPU" in proc.stderr and proc.stdout.strip() == ""


def test_bench_refuses_to_run_without_a_gpu():
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    proc = subprocess.run([sys.executable, str(ROOT / "bench.py"), "--steps", "1", "--warmup", "0"], capture_output=True,
                          text=True, timeout=300)
    assert proc.returncode != 0 and proc.stdout.strip() == ""  # no CPU fallback, no JSON line


def test_every_recorded_traffic_figure_names_a_workload_and_a_committed_profile_summary():
    import importlib.util

    spec = importlib.util.spec_from_file_location("bench_module", ROOT / "bench.py")
    bench = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(bench)
    known = (set(workloads.DECODE_CONFIGS) | set(workloads.CACHING_CONFIGS) | set(workloads.KV_CACHING_CONFIGS)
             | set(workloads.ROPE_CACHING_CONFIGS) | set(workloads.PREFILL_CONFIGS))
    for name, (nbytes, summary, commit) in bench.MEASURED_TRAFFIC.items():
        assert name in known
        assert nbytes > 0 and len(commit) >= 7
        text = (ROOT / "profiles" / summary).read_text()
        assert "FETCH_SIZE" in text and "rocprofv3 --pmc" in text
        fields = bench.traffic_fields(name)
        assert fields["traffic"] == nbytes and fields["traffic_profile"] == "profiles/" + summary
        assert fields["traffic_commit"] == commit
        assert all(not isinstance(v, (dict, list)) for v in fields.values())  # flat: scalars only
    assert bench.traffic_fields("no_such_workload") == {"traffic": None, "traffic_profile": None, "traffic_commit": None}


@pytest.mark.parametrize("name", sorted(workloads.DECODE_CONFIGS))
def test_decode_workloads_are_reproducible_and_consistent(name):
    cfg = workloads.DECODE_CONFIGS[name]
    lens = workloads.draw_seq_lens(cfg)
    assert np.array_equal(lens, workloads.draw_seq_lens(cfg))
    assert lens.min() >= cfg.min_len and lens.max() <= cfg.max_len and len(lens) == cfg.num_seqs
    e = 2
    kv = int(lens.sum()) * cfg.num_kv_heads * (cfg.head_size + cfg.v_size) * e
    total = workloads.decode_algorithmic_bytes(cfg, lens)
    assert kv < total < kv * 1.10 + 1_000_000  # K and V once, plus query, output, table entries and lengths


def test_c1_inputs_match_their_description():
    """fp16, batch 4, 8 query = 8 KV heads, head 128, pages of 16, lengths in [1, 256], pool of exactly the
    pages needed, dealt by a permutation."""
    cfg = workloads.DECODE_CONFIGS["c1_plumbing_mha"]
    inp = workloads.make_decode_inputs(cfg)
    blocks = (inp.seq_lens + 15) // 16
    assert inp.q.shape == (4, 8, 128) and inp.q.dtype == torch.float16
    assert inp.k_cache.shape == (int(blocks.sum()), 8, 16, 128) == inp.v_cache.shape
    used = torch.cat([inp.block_tables[b, :int(blocks[b])] for b in range(4)])
    assert sorted(used.tolist()) == list(range(int(blocks.sum())))  # every page used exactly once
    assert inp.scale == pytest.approx(128 ** -0.5)
    again = workloads.make_decode_inputs(cfg)
    assert torch.equal(again.q, inp.q) and torch.equal(again.block_tables, inp.block_tables)


def test_latent_attention_workload_shapes():
    cfg = workloads.DECODE_CONFIGS["m1_mla_16_heads_b32"]
    assert (cfg.head_size, cfg.v_size, cfg.num_kv_heads) == (576, 512, 1)
    small = workloads.DecodeConfig("t", torch.bfloat16, 2, 16, 1, 576, 16, 1, 40, seed=1, value_size=512)
    inp = workloads.make_decode_inputs(small)
    assert inp.k_cache.shape[-1] == 576 and inp.v_cache.shape[-1] == 512 and inp.q.shape[-1] == 576


def test_caching_workload_accounting():
    cfg = workloads.CACHING_CONFIGS["c5_prefill_scatter"]
    inp = workloads.make_caching_inputs(cfg)
    slots = inp.slot_mapping.numpy()
    valid = slots[slots >= 0]
    assert len(np.unique(valid)) == len(valid) and valid.max() < cfg.num_slots
    assert 0.03 < (slots < 0).mean() < 0.07
    assert workloads.caching_algorithmic_bytes(cfg, slots) == 2 * len(valid) * 8 * 128 * 2 * 2 + 4096 * 8


def test_kv_caching_workload_accounting():
    cfg = workloads.KV_CACHING_CONFIGS["k2_append_prefill_chunk"]
    assert workloads.kv_caching_algorithmic_bytes(cfg) == 2 * (8 * 8 * 512 * 128 * 2 * 2) + 8 * 8
    small = workloads.KVCachingConfig("t", torch.float16, 3, 2, 32, 5, 16, seed=2)
    inp = workloads.make_kv_caching_inputs(small)
    assert inp.k.shape == (3, 2, 5, 16) and inp.k_cache.shape == (3, 2, 32, 16)
    assert int(inp.past_kv_lengths.max()) + 5 <= 32 and int(inp.past_kv_lengths.min()) >= 0


def test_prefill_flops_count_visible_pairs():
    cfg = workloads.PrefillConfig("t", torch.bfloat16, 2, 4, 2, 128, 16, 3, 3, 10, 10, seed=3)
    new, history = workloads.draw_prefill_lens(cfg)
    assert new.tolist() == [3, 3] and history.tolist() == [10, 10]
    pairs = 2 * (11 + 12 + 13)
    assert workloads.prefill_flops(cfg, new, history) == pairs * 4 * 4 * 128
