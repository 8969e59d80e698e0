"""Pins of the page_attention oracle (``oracle/page_attention_oracle.py``) -- CPU only."""

import numpy as np
import pytest

from oracle import rpa_oracle
from oracle.page_attention_oracle import page_attention_exact, page_attention_strict, to_interleaved


def bf(x):
    return rpa_oracle.bf16_round(np.asarray(x, dtype=np.float32))


def make(rng, ctx, Hq=4, Hkv=2, D=16, bs=4, max_blocks=None, R=bf):
    S = len(ctx)
    max_blocks = max_blocks or -(-max(ctx) // bs) + 1
    nb = S * max_blocks + 2
    q = R(rng.standard_normal((S, Hq, D)))
    kc = R(rng.standard_normal((nb, Hkv, bs, D)))
    vc = R(rng.standard_normal((nb, Hkv, bs, D)))
    bt = rng.permutation(nb)[: S * max_blocks].reshape(S, max_blocks).astype(np.int32)
    return q, kc, vc, np.asarray(ctx, np.int32), bt


def brute(q, kc, vc, ctx, bt, scale):
    S, Hq, D = q.shape
    Hkv, bs = kc.shape[1], kc.shape[2]
    G = Hq // Hkv
    out = np.zeros((S, Hq, D))
    for s in range(S):
        for h in range(Hq):
            j = h // G
            logits = []
            for t in range(int(ctx[s])):
                logits.append(float(np.dot(q[s, h].astype(np.float64), kc[bt[s, t // bs], j, t % bs].astype(np.float64))) * scale)
            m = max(logits)
            w = [np.exp(x - m) for x in logits]
            z = sum(w)
            for t in range(int(ctx[s])):
                out[s, h] += w[t] / z * vc[bt[s, t // bs], j, t % bs]
    return out


@pytest.mark.parametrize("seed", range(4))
def test_exact_against_brute_force(seed):
    rng = np.random.default_rng(seed)
    ctx = [int(rng.integers(1, 14)) for _ in range(3)]
    args = make(rng, ctx, bs=int(rng.choice([1, 2, 4])))
    np.testing.assert_allclose(page_attention_exact(*args, attn_scale=0.3), brute(*args, 0.3), rtol=1e-12, atol=1e-12)


def test_one_key_returns_its_value_row_and_zero_query_the_mean():
    rng = np.random.default_rng(1)
    q, kc, vc, ctx, bt = make(rng, [1, 7], Hq=4, Hkv=2, bs=4)
    out = page_attention_strict(q, kc, vc, ctx, bt, attn_scale=0.25)
    assert np.array_equal(out[0], np.repeat(vc[bt[0, 0], :, 0], 2, axis=0))
    q0 = np.zeros_like(q)
    out0 = page_attention_exact(q0, kc, vc, ctx, bt)
    rows = np.stack([vc[bt[1, t // 4], :, t % 4] for t in range(7)]).astype(np.float64)  # [7, Hkv, D]
    np.testing.assert_allclose(out0[1], np.repeat(rows.mean(axis=0), 2, axis=0), rtol=1e-12)


def test_strict_is_within_tolerance_of_exact_in_both_dtype_modes():
    rng = np.random.default_rng(3)
    args = make(rng, [5, 33, 64, 17], Hq=8, Hkv=2, D=64, bs=8)
    exact = page_attention_exact(*args, attn_scale=0.125)
    d = np.abs(page_attention_strict(*args, attn_scale=0.125) - exact)
    assert d.max() < 2e-2 and d.mean() < 2e-3
    d32 = np.abs(page_attention_strict(*args, attn_scale=None) - page_attention_exact(*args))
    assert d32.max() < 1e-5


def test_block_permutation_invariance():
    rng = np.random.default_rng(4)
    q, kc, vc, ctx, bt = make(rng, [9, 14], bs=4)
    perm = rng.permutation(kc.shape[0])
    inv = np.empty_like(perm)
    inv[perm] = np.arange(len(perm))
    a = page_attention_strict(q, kc, vc, ctx, bt, attn_scale=0.2)
    b = page_attention_strict(q, kc[perm], vc[perm], ctx, inv[bt].astype(np.int32), attn_scale=0.2)
    assert np.array_equal(a, b)


def test_agrees_with_the_ragged_page_attention_oracle_on_one_token_per_sequence():
    """Two oracles written from two reference programs meet on their common special case."""
    rng = np.random.default_rng(6)
    q, kc, vc, ctx, bt = make(rng, [3, 12, 8], Hq=4, Hkv=2, D=16, bs=4)
    S = len(ctx)
    ref = rpa_oracle.rpa_exact(q, to_interleaved(kc, vc), ctx, bt, np.arange(S + 1, dtype=np.int32),
                               np.array([S], np.int32), softmax_scale=0.3)
    np.testing.assert_allclose(page_attention_exact(q, kc, vc, ctx, bt, attn_scale=0.3), ref[:S], rtol=1e-12, atol=1e-12)


def test_tail_entries_of_the_block_table_do_not_matter_when_the_context_is_not_empty():
    rng = np.random.default_rng(8)
    q, kc, vc, ctx, bt = make(rng, [5, 9], bs=4, max_blocks=5)
    a = page_attention_strict(q, kc, vc, ctx, bt, attn_scale=0.2)
    bt2 = bt.copy()
    bt2[0, 2:] = -1          # wraps to the last block; masked anyway
    bt2[1, 3:] = 10 ** 6     # clamped; masked anyway
    assert np.array_equal(a, page_attention_strict(q, kc, vc, ctx, bt2, attn_scale=0.2))
