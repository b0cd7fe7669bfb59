"""Writes tests/golden/c1_plumbing_mha_expected_f64.npy: the float64 two-pass-softmax result of the
small fp16 MHA plumbing configuration (4 sequences, 8 heads, head 128, lengths 1..256, shuffled block
table) on its seeded inputs. The reference holds no golden vectors for paged attention, so this
fixture comes from the independent float64 formulation in tests/exact.py - not from the oracle under
test and not from the HIP kernels. Run from the repository root: python tests/golden/make_c1_fixture.py"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from exact import exact_paged_attention  # noqa: E402
from infinicore_amd import workloads  # noqa: E402

inp = workloads.make_decode_inputs(workloads.DECODE_CONFIGS["c1_plumbing_mha"])
expected = exact_paged_attention(inp.q, inp.k_cache, inp.v_cache, inp.block_tables, inp.seq_lens, inp.scale)
np.save(Path(__file__).parent / "c1_plumbing_mha_expected_f64.npy", expected)
print("wrote", expected.shape, expected.dtype, "seq_lens", inp.seq_lens.tolist())
