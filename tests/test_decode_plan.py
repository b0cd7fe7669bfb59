"""The decode launch plan (decode_plan.h) on the host: partitions never span more block-table entries than a
wavefront holds, the work-equalising schedule is only chosen where its 32-bit tile axis fits, and the workspace
is sized for that schedule alone (the element-wise fallback is cut to fit it)."""
import ctypes
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
KNOBS = ("INFINIOP_AMD_PA_KERNEL", "INFINIOP_AMD_PA_SCHEDULE", "INFINIOP_AMD_PA_LATENT_KERNEL", "INFINIOP_AMD_PA_LATENT_HEADS",
         "INFINIOP_AMD_PA_PARTITION", "INFINIOP_AMD_PA_WAVES_PER_CU")
FIELDS = ("tiled", "balanced", "latent_wide", "partition_tokens", "max_partitions", "fallback_partition_tokens",
          "fallback_max_partitions", "waves_per_stream", "workspace_bytes", "launchable", "acc_bytes", "ml_bytes",
          "latent_chunks", "latent_roles")


def build_probe(directory):
    """Compiles tests/plan_probe.cc with the host compiler; returns plan(num_seqs, num_heads, ...) -> dict."""
    out = directory / "libplanprobe.so"
    subprocess.run(["g++", "-std=c++17", "-O1", "-shared", "-fPIC", f"-I{ROOT / 'include'}",
                    f"-I{ROOT / 'infinicore_amd' / 'csrc'}", str(ROOT / "tests" / "plan_probe.cc"), "-o", str(out)],
                   check=True, capture_output=True, text=True)
    lib = ctypes.CDLL(str(out))
    lib.planProbe.argtypes = [ctypes.POINTER(ctypes.c_longlong), ctypes.POINTER(ctypes.c_longlong)]
    lib.planProbe.restype = None

    def plan(num_seqs, num_heads, num_kv_heads, head_size, block_size, max_blocks, value_size=0, num_blocks=1 << 20,
             compute_units=256):
        args = (ctypes.c_longlong * 9)(num_seqs, num_heads, num_kv_heads, head_size, value_size or head_size, block_size,
                                      max_blocks, num_blocks, compute_units)
        res = (ctypes.c_longlong * len(FIELDS))()
        lib.planProbe(args, res)
        return dict(zip(FIELDS, res))

    return plan


@pytest.fixture(scope="module")
def probe(tmp_path_factory):
    return build_probe(tmp_path_factory.mktemp("plan"))


@pytest.fixture(autouse=True)
def no_knobs(monkeypatch):
    for k in KNOBS:
        monkeypatch.delenv(k, raising=False)


def entries_spanned(p, bs, k):
    """Block-table entries partition k (tokens [k p, (k + 1) p)) touches."""
    return ((k + 1) * p - 1) // bs - (k * p) // bs + 1


@pytest.mark.parametrize("bs", [16, 32, 64, 128, 256])
def test_partitions_fit_one_page_id_load(probe, monkeypatch, bs):
    """Every partition of the tiled kernels must lie inside 64 consecutive block-table entries, for the planned
    size, for the size grown to bound the workspace (very wide tables) and for any forced size."""
    monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", "grid")
    widths = [1, 7, 64, 513, 8129, 8130, 8160, 8161, 8192, 8097, 8184, 70000]
    for forced in (None, 16, 48, 1000, 4080, 4081, 5000, 100000):
        if forced is None:
            monkeypatch.delenv("INFINIOP_AMD_PA_PARTITION", raising=False)
        else:
            monkeypatch.setenv("INFINIOP_AMD_PA_PARTITION", str(forced))
        for width in widths:
            for heads, kv, head_size, value in ((32, 8, 128, 0), (128, 1, 576, 512), (16, 1, 576, 512)):
                pl = probe(4, heads, kv, head_size, bs, width, value_size=value)
                assert pl["tiled"]
                p = pl["partition_tokens"]
                assert pl["max_partitions"] == -(-width * bs // p)
                worst = max(entries_spanned(p, bs, k) for k in range(min(pl["max_partitions"], 4096)))
                assert worst <= 64, (bs, width, forced, p, worst)


def test_advisor_case_pages_of_64_table_of_8160(probe, monkeypatch):
    """Pages of 64 tokens, a table 8160 wide: the grown size used to be 4080 tokens (not a multiple of the
    page), whose second partition spans 65 entries."""
    monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", "grid")
    pl = probe(2, 32, 8, 128, 64, 8160)
    assert pl["partition_tokens"] % 64 == 0 and pl["partition_tokens"] <= 64 * 64


def test_work_equalising_schedule_needs_its_flat_axis_in_32_bits(probe):
    wide = probe(1024, 32, 8, 128, 16, 1 << 20)  # 1024 sequences x 2^20 tiles
    assert wide["tiled"] and not wide["balanced"]
    usual = probe(32, 32, 8, 128, 16, 256)
    assert usual["balanced"] and usual["waves_per_stream"] == 128


def test_workspace_is_that_of_the_chosen_schedule(probe):
    """c2: (128 pieces + 32 sequences) rows x 32 heads x (128 + 2) floats, plus the piece table and alignment
    slack - below the reference's 8 * B * H * (D + 2) * 4 = 4.26 MB."""
    c2 = probe(32, 32, 8, 128, 16, 256)
    rows = 128 + 32
    flags = rows * 8 * 8  # one 8-byte flag per (row, KV-head stream)
    first_tiles = 128 * 8 * 32  # 32 bytes per wavefront: where its first tiles were in the previous call
    assert c2["workspace_bytes"] == rows * 32 * 128 * 4 + 2 * rows * 32 * 4 + 256 + flags + first_tiles + 256
    assert c2["workspace_bytes"] < 8 * 32 * 32 * 130 * 4
    # the element-wise fallback (operands that are not 16-byte aligned at run time) fits the same rows
    assert c2["fallback_max_partitions"] * 32 <= rows
    assert c2["fallback_partition_tokens"] * c2["fallback_max_partitions"] >= 256 * 16
    c4 = probe(128, 64, 8, 128, 16, 512)
    assert c4["balanced"] and c4["fallback_max_partitions"] * 128 <= 128 + 128


def test_shapes_beyond_the_launch_limits_are_not_launchable(probe):
    assert probe(65535, 8, 8, 128, 16, 4)["launchable"]
    assert not probe(65536, 8, 8, 128, 16, 4)["launchable"]
    assert not probe(4, 65536, 65536, 128, 16, 4)["launchable"]


@pytest.mark.parametrize("schedule", [None, "balanced", "grid"])
def test_empty_batches_and_headless_tensors_plan_nothing(probe, monkeypatch, schedule):
    """No sequences, or no heads: a legal call that launches nothing. The plan must not divide by either count,
    whichever schedule the knob asks for."""
    if schedule:
        monkeypatch.setenv("INFINIOP_AMD_PA_SCHEDULE", schedule)
    for seqs, heads, kv in ((0, 32, 8), (4, 0, 8), (0, 0, 8)):  # (no KV heads at all is refused at validation)
        pl = probe(seqs, heads, kv, 128, 16, 256)
        assert not pl["balanced"] and pl["workspace_bytes"] >= 0


def test_four_chunks_per_workgroup_split_scores_and_values_between_wavefronts(probe, monkeypatch):
    """Latent attention with four 16-head chunks per workgroup runs the kernel whose wavefronts have roles, unless the
    knob asks for a wavefront per chunk; one chunk or eight chunks per workgroup never do."""
    def roles(num_seqs, heads):
        plan = probe(num_seqs, heads, 1, 576, 16, 256, value_size=512)
        return plan["latent_chunks"], plan["latent_roles"]
    assert roles(32, 128) == (4, 1) and roles(32, 48) == (4, 1) and roles(8, 32) == (4, 1)
    assert roles(32, 16) == (1, 0) and roles(64, 128) == (8, 0)
    monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_KERNEL", "rows")
    plan = probe(32, 128, 1, 576, 16, 256, value_size=512)
    assert (plan["latent_wide"], plan["latent_chunks"], plan["latent_roles"]) == (1, 4, 0)
    assert probe(200, 16, 1, 576, 16, 256, value_size=512)["latent_wide"] == 1  # "rows" implies the kernels on LDS tiles


def test_heads_of_576_with_values_of_576_take_the_tiled_kernel_on_two_wavefront_units(probe, monkeypatch):
    """The kernels that keep tiles in LDS are for values of 512 only, whatever the knob says; the partial results are
    sized for 576 columns."""
    for num_seqs, heads, kv in ((1, 16, 16), (32, 128, 1), (8, 40, 2)):
        plan = probe(num_seqs, heads, kv, 576, 16, 256)
        assert plan["tiled"] == 1 and plan["latent_wide"] == 0 and plan["balanced"] == 0
        assert plan["acc_bytes"] >= num_seqs * plan["max_partitions"] * heads * 576 * 4
    monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_KERNEL", "wide")
    assert probe(32, 128, 1, 576, 16, 256)["latent_wide"] == 0
    assert probe(32, 128, 1, 576, 16, 256, value_size=512)["latent_wide"] == 1


def test_head_chunks_that_share_a_latent_attention_workgroup(probe, monkeypatch):
    """One chunk of 16 heads: eight wavefronts for it (small batches) or the pairs of wavefronts; more chunks: four per
    workgroup, eight where there are more than four and at least 48 sequences x KV heads; the knob forces 64 or 128
    heads per workgroup where there is more than one chunk."""
    mla = dict(head_size=576, value_size=512, block_size=16, max_blocks=256)
    def chunks(num_seqs, heads, kv=1):
        plan = probe(num_seqs, heads, kv, mla["head_size"], mla["block_size"], mla["max_blocks"], value_size=mla["value_size"])
        return plan["latent_wide"], plan["latent_chunks"]
    assert chunks(32, 16) == (1, 1)
    assert chunks(128, 16)[0] == 0          # many sequences of one chunk: the two-wavefront units
    assert chunks(32, 32) == (1, 4) and chunks(32, 64) == (1, 4) and chunks(300, 64) == (1, 4)
    assert chunks(32, 128) == (1, 4) and chunks(47, 128) == (1, 4)
    assert chunks(48, 128) == (1, 8) and chunks(24, 256, kv=2) == (1, 8) and chunks(256, 80) == (1, 8)
    monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_HEADS", "128")
    assert chunks(4, 128) == (1, 8) and chunks(4, 32) == (1, 8) and chunks(32, 16) == (1, 1)
    monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_HEADS", "64")
    assert chunks(200, 128) == (1, 4)
    monkeypatch.setenv("INFINIOP_AMD_PA_LATENT_HEADS", "96")
    assert chunks(200, 128) == (1, 8)       # not a size the kernels have: ignored
