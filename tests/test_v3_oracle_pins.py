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


@pytest.mark.parametrize("dtype,Hkv", [("bfloat16", 2), ("float8_e4m3fn", 1)])
def test_padding_of_updated_tokens_is_zeroed_as_merge_kv_pads_it(dtype, Hkv):
    """head_dim 64 in rows of 128 and (8-bit cache, one kv head) two combined heads padded to four, the cache filled
    with non-zero values everywhere: the literal restatement scatters merge_kv's zero-padded rows (_kernel.py:44-57,
    :207-218), so an updated token's padding becomes zero and every other byte of the cache stays; the efficient
    restatement must give the same cache bit for bit."""
    rng = np.random.default_rng(21)
    q_lens, kv_lens = [3, 1, 0], [7, 9, 5]
    D, page, pps = 64, 4, 4
    pack = 2 if dtype == "bfloat16" else 4
    hx2 = -(-2 * Hkv // pack) * pack
    R = rpa_oracle._rounder(dtype)
    q, k, v, _, lens, bt, qsl, dist = make(rng, q_lens, kv_lens, Hq=4, Hkv=Hkv, D=D, page=page, pps=pps)
    k, v = R(k), R(v)
    P = 4 * pps + 3
    cache = R(1.0 + rng.random((P, page, hx2 // pack, pack, 128)).astype(np.float32))  # no zero anywhere
    kw = dict(cache_dtype=dtype, query_dtype="bfloat16")
    _, c_lit = rpa_v3_literal(q, k, v, cache, lens, bt, qsl, dist, **kw)
    _, c_fast = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, **kw)
    assert np.array_equal(c_lit, c_fast)
    rows = c_fast.reshape(P, page, hx2, 128)
    before = cache.reshape(P, page, hx2, 128)
    touched = np.zeros((P, page), bool)
    for s, (ql, kl) in enumerate(zip(q_lens, kv_lens)):
        for t in range(ql):
            pos = kl - ql + t
            touched[bt[s * pps + pos // page], pos % page] = True
    assert touched.sum() == sum(q_lens)
    assert not rows[touched][:, :, D:].any() and not rows[touched][:, 2 * Hkv:].any()
    assert np.array_equal(rows[~touched], before[~touched])


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


# ---------------------------------------------------------------- 8-bit cache (float8_e4m3fn)

def test_e4m3_rounding_agrees_with_the_cast_of_torch():
    # the restatement's rounding to float8_e4m3fn against an independent implementation of the same cast
    import torch

    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(50000).astype(np.float32) * s for s in (1e-3, 1e-2, 0.1, 1, 10, 100)]
                       + [np.array([0, 448, -448, 2.0**-9, 2.0**-10, 3 * 2.0**-10, 2.0**-6, 1.5 * 2.0**-10, 0.0625 * 17 / 16,
                                    0.0625 * 19 / 16], np.float32)])
    x = np.clip(x, -448, 448)
    ours = rpa_oracle.fp8_e4m3fn_round(x)
    theirs = torch.from_numpy(x).to(torch.float8_e4m3fn).to(torch.float32).numpy()
    assert np.array_equal(ours, theirs)
    # ties go to the even mantissa; half of the smallest subnormal goes to zero
    assert rpa_oracle.fp8_e4m3fn_round(np.float32(2.0**-10)) == 0.0
    assert rpa_oracle.fp8_e4m3fn_round(np.float32(0.0625 * 17 / 16)) == np.float32(0.0625)      # 1.0001|1 -> 1.000
    assert rpa_oracle.fp8_e4m3fn_round(np.float32(0.0625 * 19 / 16)) == np.float32(0.0625 * 1.25)  # 1.001|1 -> 1.010


def test_e5m2_rounding_agrees_with_the_cast_of_torch():
    import torch

    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(50000).astype(np.float32) * s for s in (1e-5, 1e-3, 0.1, 1, 100, 30000)]
                       + [np.array([0, 57344, -57344, 2.0**-16, 2.0**-17, 3 * 2.0**-17, 2.0**-14, 61439, 61440, 1e6, 1.125, 1.375],
                                   np.float32)])
    ours = rpa_oracle.fp8_e5m2_round(x)
    theirs = torch.from_numpy(x).to(torch.float8_e5m2).to(torch.float32).numpy()
    assert np.array_equal(ours, theirs)
    assert rpa_oracle.fp8_e5m2_round(np.float32(1.125)) == 1.0 and rpa_oracle.fp8_e5m2_round(np.float32(1.375)) == 1.5
    assert np.isinf(rpa_oracle.fp8_e5m2_round(np.float32(61440.0))) and rpa_oracle.fp8_e5m2_round(np.float32(61439.0)) == 57344.0


def test_e5m2_probabilities_are_rounded_after_normalisation():
    # as for e4m3, with this type's grid: p = 1/3 becomes 0.3125 (1.01b x 2**-2), so q = 0 over three keys returns
    # 0.3125 (v1 + v2 + v3), not their mean
    rng = np.random.default_rng(8)
    q, k, v, cache, lens, bt, qsl, dist = make(rng, [1], [3], dtype="float32", page=4, Hq=2, Hkv=2)
    f8 = rpa_oracle.fp8_e5m2_round
    P, page, hx2, _, D = cache.shape
    q, k, v, cache = bf(q) * 0, f8(k), f8(v), f8(cache).reshape(P, page, hx2 // 4, 4, D)
    out, after = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, softmax_scale=1.0, cache_dtype="float8_e5m2",
                        query_dtype="bfloat16")
    rows = after.reshape(P, page, -1, D)
    vis = np.stack([rows[bt[pos // page], pos % page] for pos in range(3)])
    for h in range(2):
        np.testing.assert_array_equal(out[0, h], bf(np.float32(0.3125) * vis[:, 2 * h + 1].sum(axis=0, dtype=np.float32)))


def make_e4m3(rng, q_lens, kv_lens, **kw):
    q, k, v, cache, lens, bt, qsl, dist = make(rng, q_lens, kv_lens, dtype="float32", **kw)
    f8 = rpa_oracle.fp8_e4m3fn_round
    P, page, hx2, _, D = cache.shape
    return bf(q), f8(k), f8(v), f8(cache).reshape(P, page, hx2 // 4, 4, D), lens, bt, qsl, dist


@pytest.mark.parametrize("seed", range(4))
def test_e4m3_efficient_restatement_agrees_with_the_literal_one(seed):
    rng = np.random.default_rng(100 + seed)
    S = int(rng.integers(1, 4))
    kv_lens = [int(rng.integers(1, 14)) for _ in range(S)]
    q_lens = [int(rng.integers(0, min(k, 5) + 1)) for k in kv_lens]
    args = make_e4m3(rng, q_lens, kv_lens, page=4)
    kw = dict(softmax_scale=0.09, cache_dtype="float8_e4m3fn", query_dtype="bfloat16")
    if seed % 2:
        kw.update(q_scale=0.03, k_scale=0.5, v_scale=2.0, sliding_window=6)
    a, ca = rpa_v3_literal(*args, **kw)
    b, cb = rpa_v3(*args, **kw)
    assert np.array_equal(ca, cb)
    np.testing.assert_allclose(a, b, atol=1e-6, rtol=0)


def test_e4m3_probabilities_are_rounded_after_normalisation():
    # q = 0: every visible key gets p = 1 / n.  n = 64: 2**-6 is representable, the output is the mean of V (exact in
    # float32: sums of multiples of 2**-15).  n = 1024: 2**-10 is half of the smallest subnormal and rounds to zero,
    # so the row is zero -- the cast of the *normalised* probabilities (_kernel.py:279) decides, not exp(s - max) = 1.
    rng = np.random.default_rng(7)
    for n, zero in ((64, False), (1024, True)):
        q, k, v, cache, lens, bt, qsl, dist = make_e4m3(rng, [1], [n], page=4, Hq=2, Hkv=2)
        q[:] = 0
        out, cache_after = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, softmax_scale=1.0, cache_dtype="float8_e4m3fn",
                                  query_dtype="bfloat16")
        if zero:
            assert not out.any()
            continue
        P, page, _, _, D = cache_after.shape
        rows = cache_after.reshape(P, page, -1, D)
        pps = bt.size // lens.shape[0]
        vis = np.stack([rows[bt[pos // page], pos % page] for pos in range(n)])  # [n, 2 Hkv, D] of sequence 0
        for h in range(2):
            np.testing.assert_array_equal(out[0, h], bf(vis[:, 2 * h + 1].astype(np.float64).mean(axis=0)))


def test_e4m3_query_is_clipped_and_cast_when_q_scale_is_given():
    # Closed form.  One query element is 100, q_scale 0.01: Q / q_scale = 10000 is clipped to 448 (_kernel.py:251-253).
    # Two keys, +1 and -1 in that element, zero elsewhere: the logits differ by 2 * 448 * softmax_scale * q_scale = ln 3,
    # so p = (0.75, 0.25), both on the e4m3 grid, and the output is 0.75 v1 + 0.25 v2.  Without the clip the
    # difference would be 24.5 and the output v1.
    rng = np.random.default_rng(9)
    q, k, v, cache, lens, bt, qsl, dist = make_e4m3(rng, [2], [2], page=4, Hq=2, Hkv=2)
    q[:] = 0
    q[1, :, 0] = 100.0   # the second token sees both keys (the first one only key 0)
    k[:] = 0
    k[0, :, 0] = 1.0
    k[1, :, 0] = -1.0
    scale = float(np.log(3.0) / (2 * 448 * 0.01))
    out, _ = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, softmax_scale=scale, q_scale=0.01,
                    cache_dtype="float8_e4m3fn", query_dtype="bfloat16")
    for h in range(2):
        np.testing.assert_array_equal(out[1, h], bf(0.75 * v[0, h] + 0.25 * v[1, h]))
        np.testing.assert_array_equal(out[0, h], bf(v[0, h]))


def test_slack_reports_probabilities_on_a_rounding_boundary_only():
    # Two keys whose logits differ by ln(0.40625 / 0.59375): p = (0.40625, 0.59375).  In e5m2 the first is the
    # midpoint of 0.375 and 0.4375 (step 0.0625), the second lies 0.03 from the nearest midpoint (0.5625): the row's
    # allowance is 0.0625 * max|v1|.  The first token sees one key (p = 1, exact): no allowance.
    rng = np.random.default_rng(10)
    q, k, v, cache, lens, bt, qsl, dist = make_e4m3(rng, [2], [2], page=4, Hq=2, Hkv=2)
    R = rpa_oracle._rounder("float8_e5m2")
    k, v, cache = R(k), R(v), R(cache)
    q[:] = 0
    q[1, :, 0] = 1.0
    k[:] = 0
    k[0, :, 0] = 1.0
    scale = float(np.log(0.40625 / 0.59375))
    slack = np.full((2, 2), np.nan, np.float32)
    out, _ = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, softmax_scale=scale, cache_dtype="float8_e5m2",
                    query_dtype="bfloat16", slack=slack)
    for h in range(2):
        assert slack[0, h] == 0
        assert slack[1, h] == np.float32(0.0625) * np.abs(v[0, h]).max()
        p0 = 0.375 if np.array_equal(out[1, h], bf(0.375 * v[0, h] + 0.625 * v[1, h])) else 0.4375
        np.testing.assert_array_equal(out[1, h], bf(np.float32(p0) * v[0, h] + np.float32(0.625) * v[1, h]))
    # away from every boundary the allowance is zero: p = (0.75, 0.25)
    slack[:] = np.nan
    rpa_v3(q, k, v, cache, lens, bt, qsl, dist, softmax_scale=float(np.log(3.0)), cache_dtype="float8_e5m2",
           query_dtype="bfloat16", slack=slack)
    assert not slack.any()
