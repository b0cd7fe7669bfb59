"""Seeded synthetic inputs for the paged-KV benchmark configurations (host tensors, torch CPU).

Every generator is a pure function of its seed (numpy PCG64), so the CPU container and the GPU box
build bit-identical inputs. Shapes follow the five benchmark configurations: a small MHA plumbing
case, the Llama-3-8B GQA batch-32 decode shape, a long-context peaked-softmax case, a 70B-class
one-GPU share, and a paged_caching scatter of a prefill chunk; plus prefill shapes (a small plumbing
case, whole-prompt prefill and chunked prefill over a long history at the Llama-3-8B head layout).
"""
from __future__ import annotations

from dataclasses import dataclass, field

import numpy as np
import torch


@dataclass
class DecodeConfig:
    name: str
    dtype: torch.dtype
    num_seqs: int
    num_heads: int
    num_kv_heads: int
    head_size: int
    block_size: int
    min_len: int
    max_len: int
    spare_block_fraction: float = 0.0  # extra unused pages in the pool
    peaked_fraction: float = 0.0       # fraction of token positions whose K row is scaled
    peaked_scale: float = 8.0
    seed: int = 0
    value_size: int = 0                # width of a V row; 0 = head_size (latent-attention caches: 576 / 512)

    @property
    def scale(self) -> float:
        return 1.0 / float(self.head_size) ** 0.5

    @property
    def v_size(self) -> int:
        return self.value_size or self.head_size


@dataclass
class CachingConfig:
    name: str
    dtype: torch.dtype
    num_tokens: int
    num_kv_heads: int
    head_size: int
    block_size: int
    num_slots: int
    padding_fraction: float
    seed: int = 0


@dataclass
class PrefillConfig:
    name: str
    dtype: torch.dtype
    num_seqs: int
    num_heads: int
    num_kv_heads: int
    head_size: int
    block_size: int
    min_new: int       # new (query) tokens per sequence
    max_new: int
    min_history: int   # tokens already in the cache before them
    max_history: int
    spare_block_fraction: float = 0.0
    seed: int = 0
    value_size: int = 0  # 0 = head_size

    @property
    def v_size(self) -> int:
        return self.value_size or self.head_size

    @property
    def scale(self) -> float:
        return 1.0 / float(self.head_size) ** 0.5


DECODE_CONFIGS = {
    "c1_plumbing_mha": DecodeConfig("c1_plumbing_mha", torch.float16, 4, 8, 8, 128, 16, 1, 256, seed=101),
    "c2_llama3_8b_b32": DecodeConfig("c2_llama3_8b_b32", torch.bfloat16, 32, 32, 8, 128, 16, 512, 4096,
                                     spare_block_fraction=0.10, seed=102),
    "c3_long_context": DecodeConfig("c3_long_context", torch.bfloat16, 8, 32, 8, 128, 16, 16384, 32768,
                                    peaked_fraction=0.01, seed=103),
    "c4_70b_share_b128": DecodeConfig("c4_70b_share_b128", torch.float16, 128, 64, 8, 128, 16, 1024, 8192, seed=104),
    # latent-attention cache (one KV head, 576-wide keys, 512-wide values): a tensor-parallel share of 16 query
    # heads, and all 128 heads of the model on one GPU
    "m1_mla_16_heads_b32": DecodeConfig("m1_mla_16_heads_b32", torch.bfloat16, 32, 16, 1, 576, 16, 512, 4096,
                                        spare_block_fraction=0.10, seed=106, value_size=512),
    "m2_mla_128_heads_b32": DecodeConfig("m2_mla_128_heads_b32", torch.bfloat16, 32, 128, 1, 576, 16, 512, 4096,
                                         spare_block_fraction=0.10, seed=107, value_size=512),
}
CACHING_CONFIGS = {
    "c5_prefill_scatter": CachingConfig("c5_prefill_scatter", torch.bfloat16, 4096, 8, 128, 16, 65536, 0.05, seed=105),
}


# rotary embedding of K fused with the scatter (infiniopRoPEPagedCaching): the decode step's producer (one token per
# sequence) and a prefill chunk; positions drawn from a table of 8192 rows, pairs half a vector apart (GPT-NeoX)
ROPE_CACHING_TABLE_LEN = 8192
ROPE_CACHING_CONFIGS = {
    "r1_rope_scatter_decode_step": CachingConfig("r1_rope_scatter_decode_step", torch.bfloat16, 32, 8, 128, 16, 65536, 0.0, seed=401),
    "r2_rope_scatter_prefill_chunk": CachingConfig("r2_rope_scatter_prefill_chunk", torch.bfloat16, 4096, 8, 128, 16, 65536, 0.05, seed=402),
    # the same two steps with the query (32 heads) rotated in the launch as well
    "r3_rope_qk_scatter_decode_step": CachingConfig("r3_rope_qk_scatter_decode_step", torch.bfloat16, 32, 8, 128, 16, 65536, 0.0, seed=403),
    "r4_rope_qk_scatter_prefill_chunk": CachingConfig("r4_rope_qk_scatter_prefill_chunk", torch.bfloat16, 4096, 8, 128, 16, 65536, 0.05, seed=404),
}
ROPE_QUERY_HEADS = {"r3_rope_qk_scatter_decode_step": 32, "r4_rope_qk_scatter_prefill_chunk": 32}


@dataclass
class KVCachingConfig:
    """Append to contiguous (non-paged) caches: ``new_tokens`` tokens per sequence behind random past lengths."""
    name: str
    dtype: torch.dtype
    batch: int
    num_kv_heads: int
    max_seq_len: int
    new_tokens: int
    head_size: int
    seed: int = 0


KV_CACHING_CONFIGS = {
    "k1_append_decode_step": KVCachingConfig("k1_append_decode_step", torch.bfloat16, 32, 8, 4096, 1, 128, seed=301),
    "k2_append_prefill_chunk": KVCachingConfig("k2_append_prefill_chunk", torch.bfloat16, 8, 8, 8192, 512, 128, seed=302),
}


PREFILL_CONFIGS = {
    "p1_plumbing_mha": PrefillConfig("p1_plumbing_mha", torch.float16, 4, 8, 8, 128, 16, 1, 64, 0, 128, seed=201),
    "p2_llama3_8b_prompt": PrefillConfig("p2_llama3_8b_prompt", torch.bfloat16, 4, 32, 8, 128, 16, 1024, 4096, 0, 0,
                                         spare_block_fraction=0.10, seed=202),
    "p3_llama3_8b_chunked": PrefillConfig("p3_llama3_8b_chunked", torch.bfloat16, 16, 32, 8, 128, 16, 128, 512,
                                          1024, 8192, spare_block_fraction=0.10, seed=203),
    # latent-attention cache (one KV head, keys 576, values 512), 16 query heads: chunked prefill like p3
    "p4_mla_16_heads_chunked": PrefillConfig("p4_mla_16_heads_chunked", torch.bfloat16, 16, 16, 1, 576, 16, 128, 512,
                                             1024, 8192, spare_block_fraction=0.10, seed=204, value_size=512),
}


@dataclass
class DecodeInputs:
    config: DecodeConfig
    q: torch.Tensor             # [B, H, D]
    k_cache: torch.Tensor       # [NB, Hkv, bs, D]
    v_cache: torch.Tensor
    block_tables: torch.Tensor  # [B, max_blocks] int64, unused entries 0
    seq_lens: torch.Tensor      # [B] int64
    scale: float
    extra: dict = field(default_factory=dict)


def _normal(rng: np.random.Generator, shape, dtype: torch.dtype) -> torch.Tensor:
    return torch.from_numpy(rng.standard_normal(shape, dtype=np.float32)).to(dtype)


def draw_seq_lens(cfg: DecodeConfig) -> np.ndarray:
    rng = np.random.default_rng(cfg.seed)
    return rng.integers(cfg.min_len, cfg.max_len + 1, size=cfg.num_seqs, dtype=np.int64)


def decode_algorithmic_bytes(cfg: DecodeConfig, seq_lens) -> int:
    """HBM bytes one decode call has to move: K and V once per KV head, Q in, O out, the table
    entries actually needed (int64) and the lengths."""
    e = 2
    lens = np.asarray(seq_lens, dtype=np.int64)
    kv = int(lens.sum()) * cfg.num_kv_heads * (cfg.head_size + cfg.v_size) * e
    qo = cfg.num_seqs * cfg.num_heads * (cfg.head_size + cfg.v_size) * e
    idx = int(((lens + cfg.block_size - 1) // cfg.block_size).sum()) * 8 + cfg.num_seqs * 8
    return kv + qo + idx


def make_decode_inputs(cfg: DecodeConfig, seed_offset: int = 0) -> DecodeInputs:
    """Pool of exactly the needed pages (plus the spare fraction), pages dealt to sequences by a
    seeded random permutation, Q/K/V ~ N(0,1) rounded to the storage dtype."""
    lens = draw_seq_lens(cfg)
    rng = np.random.default_rng([cfg.seed, 7, seed_offset])
    blocks_per_seq = (lens + cfg.block_size - 1) // cfg.block_size
    needed = int(blocks_per_seq.sum())
    num_blocks = int(np.ceil(needed * (1.0 + cfg.spare_block_fraction)))
    perm = rng.permutation(num_blocks)[:needed]
    max_blocks = int(blocks_per_seq.max())
    table = np.zeros((cfg.num_seqs, max_blocks), dtype=np.int64)
    cursor = 0
    for s, nb in enumerate(blocks_per_seq):
        table[s, :nb] = perm[cursor:cursor + nb]
        cursor += nb

    q = _normal(rng, (cfg.num_seqs, cfg.num_heads, cfg.head_size), cfg.dtype)
    cache_shape = (num_blocks, cfg.num_kv_heads, cfg.block_size, cfg.head_size)
    k_cache = _normal(rng, cache_shape, torch.float32)
    if cfg.peaked_fraction > 0.0:
        # scale whole token rows (all KV heads of a position) so the softmax is sharply peaked
        hot = rng.random((num_blocks, 1, cfg.block_size, 1)) < cfg.peaked_fraction
        k_cache = k_cache * torch.from_numpy(np.where(hot, cfg.peaked_scale, 1.0).astype(np.float32))
    k_cache = k_cache.to(cfg.dtype)
    v_cache = _normal(rng, cache_shape[:3] + (cfg.v_size,), cfg.dtype)
    return DecodeInputs(cfg, q, k_cache, v_cache, torch.from_numpy(table), torch.from_numpy(lens), cfg.scale)


@dataclass
class PrefillInputs:
    config: PrefillConfig
    q: torch.Tensor               # [total_q, H, D]
    k_cache: torch.Tensor         # [NB, Hkv, bs, D]
    v_cache: torch.Tensor
    block_tables: torch.Tensor    # [B, max_blocks] int64, unused entries 0
    seq_lens: torch.Tensor        # [B] int64, history + new
    cum_seq_lens_q: torch.Tensor  # [B + 1] int64
    scale: float


def draw_prefill_lens(cfg: PrefillConfig):
    rng = np.random.default_rng(cfg.seed)
    new = rng.integers(cfg.min_new, cfg.max_new + 1, size=cfg.num_seqs, dtype=np.int64)
    history = rng.integers(cfg.min_history, cfg.max_history + 1, size=cfg.num_seqs, dtype=np.int64)
    return new, history


def prefill_flops(cfg: PrefillConfig, new, history) -> int:
    """Multiply-adds x 2 of Q.K^T and P.V over the (query token, visible K/V token) pairs."""
    new, history = np.asarray(new, dtype=np.int64), np.asarray(history, dtype=np.int64)
    pairs = int((new * history + new * (new + 1) // 2).sum())
    return pairs * cfg.num_heads * 2 * (cfg.head_size + cfg.v_size)


def prefill_algorithmic_bytes(cfg: PrefillConfig, new, history) -> int:
    """Q in, O out, K and V of every sequence once per KV head, table entries and lengths."""
    e = 2
    new, history = np.asarray(new, dtype=np.int64), np.asarray(history, dtype=np.int64)
    total = new + history
    qo = int(new.sum()) * cfg.num_heads * (cfg.head_size + cfg.v_size) * e
    kv = int(total.sum()) * cfg.num_kv_heads * (cfg.head_size + cfg.v_size) * e
    idx = int(((total + cfg.block_size - 1) // cfg.block_size).sum()) * 8 + (2 * cfg.num_seqs + 1) * 8
    return qo + kv + idx


def make_prefill_inputs(cfg: PrefillConfig) -> PrefillInputs:
    """Pool of exactly the needed pages (plus the spare fraction), pages dealt to sequences by a seeded
    random permutation, Q/K/V ~ N(0,1) rounded to the storage dtype; the cache already holds the new
    tokens' K/V, as it does when the operator runs after paged_caching."""
    new, history = draw_prefill_lens(cfg)
    total = new + history
    rng = np.random.default_rng([cfg.seed, 13])
    blocks_per_seq = (total + cfg.block_size - 1) // cfg.block_size
    needed = int(blocks_per_seq.sum())
    num_blocks = int(np.ceil(needed * (1.0 + cfg.spare_block_fraction)))
    perm = rng.permutation(num_blocks)[:needed]
    table = np.zeros((cfg.num_seqs, int(blocks_per_seq.max())), dtype=np.int64)
    cursor = 0
    for s, nb in enumerate(blocks_per_seq):
        table[s, :nb] = perm[cursor:cursor + nb]
        cursor += nb
    cum = np.concatenate([[0], np.cumsum(new)]).astype(np.int64)
    q = _normal(rng, (int(cum[-1]), cfg.num_heads, cfg.head_size), cfg.dtype)
    cache_shape = (num_blocks, cfg.num_kv_heads, cfg.block_size, cfg.head_size)
    k_cache = _normal(rng, cache_shape, cfg.dtype)
    v_cache = _normal(rng, cache_shape, cfg.dtype)
    if cfg.v_size != cfg.head_size:
        v_cache = v_cache[..., :cfg.v_size].contiguous()
    return PrefillInputs(cfg, q, k_cache, v_cache, torch.from_numpy(table), torch.from_numpy(total),
                         torch.from_numpy(cum), cfg.scale)


@dataclass
class CachingInputs:
    config: CachingConfig
    k: torch.Tensor             # [ntok, Hkv, D]
    v: torch.Tensor
    k_cache: torch.Tensor       # [NB, Hkv, bs, D], pre-filled with a sentinel pattern
    v_cache: torch.Tensor
    slot_mapping: torch.Tensor  # [ntok] int64, -1 = padding


def caching_algorithmic_bytes(cfg: CachingConfig, slot_mapping) -> int:
    e = 2 if cfg.dtype in (torch.float16, torch.bfloat16) else 4
    valid = int((np.asarray(slot_mapping) >= 0).sum())
    moved = valid * cfg.num_kv_heads * cfg.head_size * e * 2  # K and V
    return 2 * moved + cfg.num_tokens * 8  # read + write + slot ids


def make_caching_inputs(cfg: CachingConfig) -> CachingInputs:
    rng = np.random.default_rng([cfg.seed, 11])
    slots = rng.permutation(cfg.num_slots)[:cfg.num_tokens].astype(np.int64)
    padding = rng.random(cfg.num_tokens) < cfg.padding_fraction
    slots[padding] = -1
    k = _normal(rng, (cfg.num_tokens, cfg.num_kv_heads, cfg.head_size), cfg.dtype)
    v = _normal(rng, (cfg.num_tokens, cfg.num_kv_heads, cfg.head_size), cfg.dtype)
    num_blocks = cfg.num_slots // cfg.block_size
    shape = (num_blocks, cfg.num_kv_heads, cfg.block_size, cfg.head_size)
    # sentinel: a value no N(0,1) draw rounds to, so untouched bytes are recognisable
    k_cache = torch.full(shape, -777.0, dtype=cfg.dtype)
    v_cache = torch.full(shape, 555.0, dtype=cfg.dtype)
    return CachingInputs(cfg, k, v, k_cache, v_cache, torch.from_numpy(slots))


def make_rope_tables(table_len: int, head_size: int, dtype: torch.dtype, theta: float = 10000.0):
    """sin / cos tables [table_len, head_size / 2] as the reference's RoPE test builds them
    (test/infiniop/rope.py:124-131)."""
    freqs = 1.0 / (theta ** (torch.arange(0, head_size, 2).float() / head_size))
    angles = torch.outer(torch.arange(table_len).float(), freqs)
    return torch.sin(angles).to(dtype), torch.cos(angles).to(dtype)


def make_rope_caching_inputs(cfg: CachingConfig):
    """The scatter's inputs plus one position per token and the tables: (CachingInputs, pos_ids, sin, cos)."""
    inp = make_caching_inputs(cfg)
    rng = np.random.default_rng([cfg.seed, 13])
    pos = torch.from_numpy(rng.integers(0, ROPE_CACHING_TABLE_LEN, cfg.num_tokens).astype(np.int64))
    sin, cos = make_rope_tables(ROPE_CACHING_TABLE_LEN, cfg.head_size, cfg.dtype)
    return inp, pos, sin, cos


def rope_caching_algorithmic_bytes(cfg: CachingConfig, slot_mapping) -> int:
    """The scatter's bytes plus one position and one row of each table per token, plus the query read once and
    written once where the workload rotates it too."""
    e = 2 if cfg.dtype in (torch.float16, torch.bfloat16) else 4
    query = 2 * cfg.num_tokens * ROPE_QUERY_HEADS.get(cfg.name, 0) * cfg.head_size * e
    return caching_algorithmic_bytes(cfg, slot_mapping) + cfg.num_tokens * (8 + 2 * (cfg.head_size // 2) * e) + query


def make_rope_query(cfg: CachingConfig):
    """The query of a workload that rotates it: [num_tokens, ROPE_QUERY_HEADS, head_size]."""
    rng = np.random.default_rng([cfg.seed, 17])
    shape = (cfg.num_tokens, ROPE_QUERY_HEADS[cfg.name], cfg.head_size)
    return torch.from_numpy(rng.standard_normal(shape, dtype=np.float32)).to(cfg.dtype)


@dataclass
class KVCachingInputs:
    config: KVCachingConfig
    k: torch.Tensor                # [B, Hkv, new_tokens, D]
    v: torch.Tensor
    k_cache: torch.Tensor          # [B, Hkv, max_seq_len, D], pre-filled with a sentinel
    v_cache: torch.Tensor
    past_kv_lengths: torch.Tensor  # [B] int64


def kv_caching_algorithmic_bytes(cfg: KVCachingConfig) -> int:
    e = 2 if cfg.dtype in (torch.float16, torch.bfloat16) else 4
    moved = cfg.batch * cfg.num_kv_heads * cfg.new_tokens * cfg.head_size * e * 2  # K and V
    return 2 * moved + cfg.batch * 8  # read + write + lengths


def make_kv_caching_inputs(cfg: KVCachingConfig) -> KVCachingInputs:
    rng = np.random.default_rng([cfg.seed, 13])
    new_shape = (cfg.batch, cfg.num_kv_heads, cfg.new_tokens, cfg.head_size)
    cache_shape = (cfg.batch, cfg.num_kv_heads, cfg.max_seq_len, cfg.head_size)
    k, v = _normal(rng, new_shape, cfg.dtype), _normal(rng, new_shape, cfg.dtype)
    past = rng.integers(0, cfg.max_seq_len - cfg.new_tokens + 1, size=cfg.batch, dtype=np.int64)
    k_cache = torch.full(cache_shape, -777.0, dtype=cfg.dtype)
    v_cache = torch.full(cache_shape, 555.0, dtype=cfg.dtype)
    return KVCachingInputs(cfg, k, v, k_cache, v_cache, torch.from_numpy(past))
