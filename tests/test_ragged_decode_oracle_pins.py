"""Pins of the ragged_decode_attention oracle (``oracle/ragged_decode_oracle.py``) -- CPU only."""

import numpy as np
import pytest

from oracle import rpa_oracle
from oracle.ragged_decode_oracle import ragged_decode_exact, ragged_decode_strict


def bf(x):
    return rpa_oracle.bf16_round(np.asarray(x, dtype=np.float32))


def make(rng, B=3, S=40, Hq=4, Hkv=2, D=16, R=bf):
    return (R(rng.standard_normal((B, Hq, D))), R(rng.standard_normal((B, S, Hkv, D))),
            R(rng.standard_normal((B, S, Hkv, D))))


def brute(q, k, v, start, end, scale, window=None, cap=None):
    B, Hq, D = q.shape
    G = Hq // k.shape[2]
    out = np.zeros((B, Hq, D))
    for b in range(B):
        for h in range(Hq):
            j = h // G
            ks = [t for t in range(int(start[b]), int(end[b]))
                  if window is None or (end[b] - 1 - window[0] <= t <= end[b] - 1 + window[1])]
            if not ks:
                continue
            lg = [float(np.dot(q[b, h].astype(np.float64), k[b, t, j].astype(np.float64))) * scale for t in ks]
            if cap is not None:
                lg = [cap * np.tanh(x / cap) for x in lg]
            m = max(lg)
            w = [np.exp(x - m) for x in lg]
            for t, wt in zip(ks, w):
                out[b, h] += wt / sum(w) * v[b, t, j]
    return out


@pytest.mark.parametrize("window,cap", [(None, None), ((5, 0), None), ((3, 2), 4.0)])
def test_exact_against_brute_force(window, cap):
    rng = np.random.default_rng(0)
    q, k, v = make(rng)
    start, end = np.array([0, 7, 12]), np.array([40, 25, 12])   # the last sequence is empty
    got = ragged_decode_exact(q, k, v, start, end, softmax_scale=0.3, sliding_window=window, logits_soft_cap=cap)
    np.testing.assert_allclose(got, brute(q, k, v, start, end, 0.3, window, cap), rtol=1e-12, atol=1e-12)
    assert not got[2].any()


def test_closed_forms():
    rng = np.random.default_rng(1)
    q, k, v = make(rng, B=2)
    # one visible key: its value row; window left = 0 keeps only the query position
    out = ragged_decode_strict(q, k, v, np.array([9, 0]), np.array([10, 33]), softmax_scale=0.25, block_size=64,
                               sliding_window=(0, 0))
    assert np.array_equal(out[0], np.repeat(v[0, 9], 2, axis=0))
    assert np.array_equal(out[1], np.repeat(v[1, 32], 2, axis=0))
    # q = 0: the mean of the visible values
    out0 = ragged_decode_exact(np.zeros_like(q), k, v, np.array([4, 0]), np.array([11, 6]))
    np.testing.assert_allclose(out0[0], np.repeat(v[0, 4:11].astype(np.float64).mean(axis=0), 2, axis=0), rtol=1e-12)


def test_strict_is_within_tolerance_of_exact_when_one_block_covers_the_sequence():
    rng = np.random.default_rng(2)
    q, k, v = make(rng, B=4, S=300, Hq=8, Hkv=2, D=64)
    start, end = np.array([0, 3, 0, 10]), np.array([300, 200, 17, 129])
    exact = ragged_decode_exact(q, k, v, start, end, softmax_scale=0.125)
    d = np.abs(ragged_decode_strict(q, k, v, start, end, softmax_scale=0.125, block_size=512) - exact)
    assert d.max() < 2e-2 and d.mean() < 2e-3, (d.max(), d.mean())


def test_the_reference_recurrence_is_not_attention_once_a_sequence_spans_several_blocks():
    """``o_curr`` is already divided by the new normaliser (``attn_weights = exp_scores / l_new``, :188-189) and
    is then weighted by ``l_curr / l_new`` again (:191), so every block after the first is under-weighted.  The
    restatement keeps that; sequences inside one block are unaffected."""
    rng = np.random.default_rng(2)
    q, k, v = make(rng, B=2, S=300, Hq=8, Hkv=2, D=64)
    start, end = np.array([0, 0]), np.array([300, 17])
    exact = ragged_decode_exact(q, k, v, start, end, softmax_scale=0.125)
    strict = ragged_decode_strict(q, k, v, start, end, softmax_scale=0.125, block_size=32)
    assert np.abs(strict[0] - exact[0]).max() > 0.05          # 10 blocks
    assert np.abs(strict[1] - exact[1]).max() < 2e-2          # 17 keys: one block
    # with the block's numerator left un-normalised the same scan is attention again
    fixed = _scan_with_the_numerator_not_normalised(q[0], k[0], v[0], 300, 0.125, 32)
    np.testing.assert_allclose(fixed, exact[0], rtol=1e-9, atol=1e-9)


def _scan_with_the_numerator_not_normalised(q, k, v, end, scale, bs):
    Hq, D = q.shape
    Hkv = k.shape[1]
    G = Hq // Hkv
    qs = q.reshape(Hkv, G, D).astype(np.float64) * scale
    o = np.zeros((Hkv, G, D))
    m = np.full((Hkv, G, 1), -np.inf)
    l = np.zeros((Hkv, G, 1))
    for i in range(0, end, bs):
        kb = k[i:min(i + bs, end)].transpose(1, 0, 2).astype(np.float64)
        vb = v[i:min(i + bs, end)].transpose(1, 0, 2).astype(np.float64)
        sc = np.einsum("jgd,jkd->jgk", qs, kb)
        m_new = np.maximum(m, sc.max(axis=-1, keepdims=True))
        e = np.exp(sc - m_new)
        corr = np.exp(m - m_new)
        l_new = corr * l + e.sum(axis=-1, keepdims=True)
        o = (corr * l * o + np.einsum("jgk,jkd->jgd", e, vb)) / l_new
        m, l = m_new, l_new
    return o.reshape(Hq, D)


def test_the_reference_turns_nan_when_its_first_block_has_no_visible_key():
    rng = np.random.default_rng(3)
    q, k, v = make(rng, B=2, S=64)
    out = ragged_decode_strict(q, k, v, np.array([16, 0]), np.array([40, 40]), softmax_scale=0.2, block_size=16)
    assert np.isnan(out[0]).all() and np.isfinite(out[1]).all()
    out = ragged_decode_strict(q, k, v, np.array([0, 0]), np.array([40, 12]), softmax_scale=0.2, block_size=16,
                               sliding_window=(7, 0))
    assert np.isnan(out[0]).all() and np.isfinite(out[1]).all()


def test_agrees_with_the_ragged_page_attention_oracle_on_one_page_per_sequence():
    rng = np.random.default_rng(4)
    B, S, Hkv, D = 3, 16, 2, 16
    q, k, v = make(rng, B=B, S=S, Hkv=Hkv, D=D)
    end = np.array([16, 5, 11], np.int32)
    pages = np.stack([k, v], axis=3).reshape(B, S, 2 * Hkv, D)     # page b = sequence b, K at 2j, V at 2j + 1
    ref = rpa_oracle.rpa_exact(q, pages, end, np.arange(B, dtype=np.int32)[:, None], np.arange(B + 1, dtype=np.int32),
                               np.array([B], np.int32), softmax_scale=0.3, sliding_window=4)
    got = ragged_decode_exact(q, k, v, np.zeros(B, np.int32), end, softmax_scale=0.3, sliding_window=(3, 0))
    np.testing.assert_allclose(got, ref[:B], rtol=1e-12, atol=1e-12)
