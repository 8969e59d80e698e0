"""Algorithmic work of a ragged paged attention batch and the MI355X peaks it is priced against."""

from __future__ import annotations

import numpy as np

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, GB/s
MFMA_BF16_PEAK_TFLOPS = 2500.0  # dense bf16 MFMA, TFLOP/s


def algorithmic_counts(q_lens, kv_lens, *, num_q_heads, num_kv_heads, head_dim, page_size, sliding_window=None,
                       elem_bytes=2) -> dict:
    """Minimum FLOPs and HBM bytes of one forward pass.

    ``flops = 4 * D * Hq * sum over rows of visible keys`` (QK^T and PV at 2 flop per MAC).
    ``bytes``: every K/V token a sequence can see is read once per kv head
    (``min(kv_len, q_len + window - 1)`` tokens with a sliding window), Q is read once, O is
    written once, plus the int32 metadata (block-table entries in use, lengths, offsets).
    """
    q_lens = np.asarray(q_lens, dtype=np.int64)
    kv_lens = np.asarray(kv_lens, dtype=np.int64)
    pairs = kv_tokens = pages = 0
    for q_len, kv_len in zip(q_lens.tolist(), kv_lens.tolist()):
        if q_len <= 0:
            continue
        vis = (kv_len - q_len) + np.arange(q_len, dtype=np.int64) + 1
        e = kv_len
        if sliding_window is not None:
            vis = np.minimum(vis, int(sliding_window))
            e = min(kv_len, q_len + int(sliding_window) - 1)
        pairs += int(vis.sum())
        kv_tokens += e
        pages += -(-e // page_size)
    tokens = int(q_lens.sum())
    kv_bytes = kv_tokens * 2 * num_kv_heads * head_dim * elem_bytes
    qo_bytes = 2 * tokens * num_q_heads * head_dim * elem_bytes
    meta_bytes = 4 * (pages + 2 * len(q_lens) + 1)
    return dict(flops=4 * head_dim * num_q_heads * pairs, kv_bytes=kv_bytes, qo_bytes=qo_bytes,
                meta_bytes=meta_bytes, bytes=kv_bytes + qo_bytes + meta_bytes, tokens=tokens, pairs=pairs)
