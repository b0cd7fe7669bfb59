"""An independent statement of paged attention used to pin the oracle: gather the sequence's tokens
through the block table, then the textbook two-pass softmax in float64 (numpy). It shares no code and
no formulation with oracle/paged_oracle.c (no online recurrence, no log2 domain, no epsilon)."""
import numpy as np
import torch


def gather_sequence(cache: torch.Tensor, table_row, length: int) -> np.ndarray:
    """[length, num_kv_heads, d] float64 rows of one sequence."""
    block_size = cache.shape[2]
    pos = np.arange(length)
    pages = np.asarray(table_row, dtype=np.int64)[pos // block_size]
    return cache[torch.from_numpy(pages), :, torch.from_numpy(pos % block_size), :].to(torch.float64).numpy()


def exact_paged_attention(q, k_cache, v_cache, block_tables, seq_lens, scale, alibi_slopes=None) -> np.ndarray:
    """float64 [num_seqs, num_heads, value_size]; rows of empty sequences are NaN."""
    B, H, _ = q.shape
    Hkv = k_cache.shape[1]
    group = H // Hkv
    out = np.full((B, H, v_cache.shape[3]), np.nan)
    qd = q.to(torch.float64).numpy()
    for s in range(B):
        L = int(seq_lens[s])
        if L <= 0:
            continue
        K = gather_sequence(k_cache, block_tables[s], L)
        V = gather_sequence(v_cache, block_tables[s], L)
        for h in range(H):
            logits = float(scale) * (K[:, h // group, :] @ qd[s, h])
            if alibi_slopes is not None:
                logits = logits + float(alibi_slopes[h]) * (np.arange(L) - (L - 1))
            p = np.exp(logits - logits.max())
            out[s, h] = (p / p.sum()) @ V[:, h // group, :]
    return out


def ulp(dtype: torch.dtype, magnitude: np.ndarray) -> np.ndarray:
    """Spacing of `dtype` at |magnitude| (normal range)."""
    bits = 10 if dtype == torch.float16 else 7
    m = np.maximum(np.abs(magnitude), 2.0 ** -14)
    return 2.0 ** (np.floor(np.log2(m)) - bits)
