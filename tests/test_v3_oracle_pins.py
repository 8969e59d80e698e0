"""Pins of the v3 oracle (``oracle/rpa_v3_oracle.py``) -- CPU only.

The efficient restatement is checked against the step-by-step one, the cache update against a closed form, the
attention against the float64 dense oracle of the v2 operation on the updated cache, and against closed forms.
"""

import numpy as np
import pytest

from oracle import rpa_oracle
from oracle.rpa_v3_oracle import merge_kv, rpa_v3, rpa_v3_literal


def bf(x):
    return rpa_oracle.bf16_round(np.asarray(x, dtype=np.float32))


def make(rng, q_lens, kv_lens, Hq=4, Hkv=2, D=128, page=4, pps=None, extra_seqs=1, dtype="bfloat16"):
    S = len(q_lens)
    max_seqs = S + extra_seqs
    pps = pps or -(-max(kv_lens) // page) + 1
    P = max_seqs * pps + 3
    R = bf if dtype == "bfloat16" else (lambda a: np.asarray(a, np.float32))
    T = int(sum(q_lens)) + 3
    pack = 2 if dtype == "bfloat16" else 1
    q = R(rng.standard_normal((T, Hq, D)))
    k = R(rng.standard_normal((T, Hkv, D)))
    v = R(rng.standard_normal((T, Hkv, D)))
    cache = R(rng.standard_normal((P, page, 2 * Hkv // pack, pack, D)))
    bt = rng.permutation(P)[: max_seqs * pps].astype(np.int32)
    lens = np.zeros(max_seqs, np.int32)
    lens[:S] = kv_lens
    qsl = np.zeros(max_seqs + 1, np.int32)
    qsl[1:S + 1] = np.cumsum(q_lens)
    qsl[S + 1:] = qsl[S]
    dist = np.array([0, 0, S], np.int32)
    return q, k, v, cache, lens, bt, qsl, dist


def test_merge_kv_interleaves_k_and_v_rows():
    # _kernel.py:44-57: K of kv head j is combined row 2j, V row 2j + 1; at D % 128 == 0 nothing is padded
    T, Hkv, D = 3, 2, 128
    k = np.arange(T * Hkv * D, dtype=np.float32).reshape(T, Hkv, D)
    v = -k - 1
    m = merge_kv(k, v, "bfloat16").reshape(T, 2 * Hkv, D)
    for j in range(Hkv):
        assert np.array_equal(m[:, 2 * j], k[:, j]) and np.array_equal(m[:, 2 * j + 1], v[:, j])
    # D = 64 is padded to 128 with zeros, an odd combined head count is impossible (2 * Hkv)
    m64 = merge_kv(k[:, :, :64], v[:, :, :64], "float32")
    assert m64.shape == (T, 2 * Hkv, 1, 128) and not m64[..., 64:].any()


@pytest.mark.parametrize("seed", range(6))
def test_efficient_restatement_agrees_with_the_literal_one(seed):
    rng = np.random.default_rng(seed)
    S = int(rng.integers(1, 4))
    kv_lens = [int(rng.integers(1, 14)) for _ in range(S)]
    q_lens = [int(rng.integers(0, min(k, 5) + 1)) for k in kv_lens]
    args = make(rng, q_lens, kv_lens, page=int(rng.choice([2, 4])))
    kw = dict(softmax_scale=0.09)
    if seed % 3 == 1:
        kw["sliding_window"] = 3
    if seed % 3 == 2:
        kw.update(logits_soft_cap=5.0, k_scale=0.5, v_scale=2.0, q_scale=4.0)
    o1, c1 = rpa_v3_literal(*args, **kw)
    o2, c2 = rpa_v3(*args, **kw)
    assert np.array_equal(c1, c2)
    np.testing.assert_allclose(o2, o1, atol=2 ** -8, rtol=2 ** -7)  # both rounded to bf16; summation order differs
    assert np.mean(o1 != o2) < 0.02


def test_cache_update_closed_form():
    rng = np.random.default_rng(11)
    q_lens, kv_lens = [3, 1, 0], [7, 9, 5]
    q, k, v, cache, lens, bt, qsl, dist = make(rng, q_lens, kv_lens, page=4, pps=4)
    _, new = rpa_v3(q, k, v, cache, lens, bt, qsl, dist)
    expect = cache.copy().reshape(cache.shape[0], cache.shape[1], -1, cache.shape[-1])
    for s, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        for t in range(ql):
            pos = kl - ql + t
            page = bt[s * 4 + pos // 4]
            expect[page, pos % 4, 0::2] = k[qsl[s] + t]
            expect[page, pos % 4, 1::2] = v[qsl[s] + t]
    assert np.array_equal(new.reshape(expect.shape), expect)
    assert (new != cache).any()


@pytest.mark.parametrize("window,cap", [(None, None), (5, None), (None, 8.0)])
def test_attention_matches_the_dense_float64_oracle_on_the_updated_cache(window, cap):
    rng = np.random.default_rng(5)
    q_lens, kv_lens = [4, 1, 6], [11, 13, 6]
    q, k, v, cache, lens, bt, qsl, dist = make(rng, q_lens, kv_lens, page=4, pps=4)
    out, new = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, softmax_scale=0.11, sliding_window=window,
                      logits_soft_cap=cap)
    P, page, _, _, D = new.shape
    ref = rpa_oracle.rpa_exact(q, new.reshape(P, page, -1, D), lens, bt.reshape(len(lens), -1), qsl,
                               np.array([3], np.int32), softmax_scale=0.11, sliding_window=window, logits_soft_cap=cap)
    total = int(qsl[3])
    assert np.abs(out[:total] - ref[:total]).max() < 2e-2  # out is bf16, P is bf16
    assert not out[total:].any()


def test_zero_queries_give_the_mean_of_the_visible_values_including_the_new_tokens():
    rng = np.random.default_rng(2)
    q_lens, kv_lens = [3], [6]
    q, k, v, cache, lens, bt, qsl, dist = make(rng, q_lens, kv_lens, Hq=2, Hkv=1, page=2, pps=4, dtype="float32")
    q[:] = 0
    out, new = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, cache_dtype="float32")
    rows = new.reshape(new.shape[0], 2, 2, -1)
    vals = np.stack([rows[bt[pos // 2], pos % 2, 1] for pos in range(6)])  # V rows in position order
    assert np.array_equal(vals[3:], v[:3, 0])                          # the new tokens are positions 3, 4, 5
    for i in range(3):
        np.testing.assert_allclose(out[i, 0], vals[: 3 + i + 1].mean(axis=0), rtol=1e-6, atol=1e-6)


def test_scales_fold_as_the_reference_composes_them():
    # S * k_scale, O * v_scale; q / q_scale then S * q_scale cancels up to the rounding of q / q_scale (exact for powers of two)
    rng = np.random.default_rng(9)
    args = make(rng, [2, 1], [5, 4])
    base, _ = rpa_v3(*args, softmax_scale=0.1)
    a, _ = rpa_v3(*args, softmax_scale=0.05, k_scale=2.0)
    b, _ = rpa_v3(*args, softmax_scale=0.1, q_scale=4.0)
    c, _ = rpa_v3(*args, softmax_scale=0.1, v_scale=2.0)
    assert np.array_equal(a, base) and np.array_equal(b, base)
    np.testing.assert_allclose(c, 2 * base, rtol=2 ** -7)
