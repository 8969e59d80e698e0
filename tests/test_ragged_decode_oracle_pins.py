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


# ---- attention sinks (softmax_aux): _xla_impl_fwd.py:71-75 (mask) and :98-134 (bias)

def brute_sinks(q, k, v, start, end, scale, aux, window=None, cap=None):
    """Key by key, from the program's two rules: [start, start + ns) always visible, bias on absolute t < ns."""
    B, Hq, D = q.shape
    S = k.shape[1]
    G = Hq // k.shape[2]
    aux = np.asarray(aux, dtype=np.float64)
    ns = aux.shape[-1]
    out = np.zeros((B, Hq, D))
    for b in range(B):
        for h in range(Hq):
            j, g = h // G, h % G
            row = aux if aux.ndim == 1 else aux[g if aux.shape[0] > 1 else 0]
            ks = []
            for t in range(S):
                seen = start[b] <= t < end[b]
                if window is not None:
                    seen = seen and (end[b] - 1 - window[0] <= t <= end[b] - 1 + window[1])
                if seen or start[b] <= t < start[b] + ns:
                    ks.append(t)
            if not ks:
                continue
            lg = []
            for t in ks:
                x = float(np.dot(q[b, h].astype(np.float64), k[b, t, j].astype(np.float64))) * scale
                if cap is not None:
                    x = cap * np.tanh(x / cap)
                lg.append(x + (row[t] if t < ns else 0.0))
            m = max(lg)
            w = [np.exp(x - m) for x in lg]
            for t, wt in zip(ks, w):
                out[b, h] += wt / sum(w) * v[b, t, j]
    return out


@pytest.mark.parametrize("window,cap", [(None, None), ((4, 0), None), ((2, 1), 3.0)])
@pytest.mark.parametrize("aux_shape", ["vector", "one_row", "per_group_head"])
def test_exact_with_sinks_against_brute_force(window, cap, aux_shape):
    rng = np.random.default_rng(5)
    q, k, v = make(rng, B=5)
    # sequence 1 starts past the biased positions, 2 is empty, 3 has its sink range running past `end`,
    # 4 has it cut by seq_len
    start, end = np.array([0, 7, 12, 20, 38]), np.array([40, 25, 12, 21, 40])
    aux = {"vector": rng.standard_normal(3), "one_row": rng.standard_normal((1, 3)),
           "per_group_head": rng.standard_normal((2, 3))}[aux_shape].astype(np.float32)  # the oracle keeps float32
    got = ragged_decode_exact(q, k, v, start, end, softmax_scale=0.3, sliding_window=window, logits_soft_cap=cap,
                              softmax_aux=aux)
    np.testing.assert_allclose(got, brute_sinks(q, k, v, start, end, 0.3, aux, window, cap), rtol=1e-11, atol=1e-12)
    # the empty sequence attends to its sink range alone
    assert got[2].any()


def test_sink_closed_forms():
    rng = np.random.default_rng(6)
    q, k, v = make(rng, B=1, S=32, Hq=2, Hkv=1, D=8)
    v64 = v.astype(np.float64)
    zero = np.zeros_like(q)
    # q = 0, window keeps only the query position 19: the visible keys are 19 and the sink range {0, 1}, the sink
    # logits are the biases themselves -> weights e^a0, e^a1, 1 (biases exact in float32)
    a = np.array([0.75, -0.5])
    out = ragged_decode_exact(zero, k, v, np.array([0]), np.array([20]), sliding_window=(0, 0), softmax_aux=a)
    w = np.array([np.exp(0.75), np.exp(-0.5), 1.0])
    want = (w[0] * v64[0, 0, 0] + w[1] * v64[0, 1, 0] + w[2] * v64[0, 19, 0]) / w.sum()
    np.testing.assert_allclose(out[0, 0], want, rtol=1e-12)
    # a sequence that starts at 5: its sink range is {5, 6}, which lies past the biased positions {0, 1}, so the
    # biases do not matter and the three visible keys weigh the same
    out = ragged_decode_exact(zero, k, v, np.array([5]), np.array([20]), sliding_window=(0, 0), softmax_aux=a)
    np.testing.assert_allclose(out[0, 1], (v64[0, 5, 0] + v64[0, 6, 0] + v64[0, 19, 0]) / 3.0, rtol=1e-12)
    # ... but a sequence starting at 1 has key 1 both in its sink range and biased, key 2 in the range only
    out = ragged_decode_exact(zero, k, v, np.array([1]), np.array([20]), sliding_window=(0, 0), softmax_aux=a)
    want = (np.exp(-0.5) * v64[0, 1, 0] + v64[0, 2, 0] + v64[0, 19, 0]) / (np.exp(-0.5) + 2.0)
    np.testing.assert_allclose(out[0, 0], want, rtol=1e-12)
    # the range is not cut at `end`: end = start + 1 still sees start + 1
    out = ragged_decode_exact(zero, k, v, np.array([8]), np.array([9]), softmax_aux=a)
    np.testing.assert_allclose(out[0, 0], (v64[0, 8, 0] + v64[0, 9, 0]) / 2.0, rtol=1e-12)
    # zero biases inside the plain range change nothing
    full = ragged_decode_exact(q, k, v, np.array([3]), np.array([30]), softmax_scale=0.4)
    same = ragged_decode_exact(q, k, v, np.array([3]), np.array([30]), softmax_scale=0.4, softmax_aux=np.zeros(4))
    np.testing.assert_allclose(same, full, rtol=1e-13)
    # the bias comes after the soft cap: with a tiny cap the logits of the keys vanish, the bias does not
    out = ragged_decode_exact(q, k, v, np.array([0]), np.array([2]), softmax_scale=0.4, logits_soft_cap=1e-9,
                              softmax_aux=np.array([2.0]))
    want = (np.exp(2.0) * v64[0, 0, 0] + v64[0, 1, 0]) / (np.exp(2.0) + 1.0)
    np.testing.assert_allclose(out[0, 1], want, rtol=1e-6)


def test_sink_rows_follow_the_program_s_broadcast():
    rng = np.random.default_rng(7)
    q, k, v = make(rng, B=1, S=16, Hq=6, Hkv=2, D=8)   # G = 3
    start, end = np.array([0]), np.array([16])
    per_head = rng.standard_normal((3, 2)).astype(np.float32)
    out = ragged_decode_exact(q, k, v, start, end, softmax_aux=per_head)
    # row g serves the g-th query head of every kv head: heads 1 and 4 share row 1
    for h in (1, 4):
        alone = ragged_decode_exact(q[:, h:h + 1], k[:, :, h // 3:h // 3 + 1], v[:, :, h // 3:h // 3 + 1], start, end,
                                    softmax_aux=per_head[1])
        np.testing.assert_allclose(out[0, h], alone[0, 0], rtol=1e-12)
    # [num_kv_heads, num_sinks] = [2, 2] does not broadcast against G = 3
    with pytest.raises(ValueError):
        ragged_decode_exact(q, k, v, start, end, softmax_aux=np.zeros((2, 2)))


def test_strict_with_sinks_is_within_tolerance_of_exact_when_one_block_covers_the_sequence():
    rng = np.random.default_rng(8)
    q, k, v = make(rng, B=4, S=96, Hq=8, Hkv=2, D=32)
    start, end = np.array([0, 2, 30, 50]), np.array([96, 70, 64, 50])
    aux = rng.standard_normal((4, 4)).astype(np.float32)
    for window in (None, (7, 0)):
        want = ragged_decode_exact(q, k, v, start, end, sliding_window=window, softmax_aux=aux)
        for aux_dtype in ("float32", "bfloat16"):
            a = aux if aux_dtype == "float32" else bf(aux)
            got = ragged_decode_strict(q, k, v, start, end, block_size=128, sliding_window=window, softmax_aux=a,
                                       aux_dtype=aux_dtype)
            w = want if aux_dtype == "float32" else ragged_decode_exact(q, k, v, start, end, sliding_window=window,
                                                                        softmax_aux=a)
            err = np.abs(got - w)
            assert err.max() <= 2e-2 and err.mean() <= 2e-3
