"""Pins the CPU oracle without the reference at hand.

The reference's tests hold no golden vectors for its XLA ragged paged attention and the
reference cannot be imported here, so ``oracle.rpa_oracle`` is pinned by what the
mathematics fixes: closed forms, invariants, the contiguous special case against a
library SDPA, and a scalar brute force.  Each check is chosen so that one plausible
mistake (wrong page / slot / head index, K and V swapped, off-by-one in the causal or
window mask, cap applied after the mask, a dropped sink term) fails it.
"""

import math

import numpy as np
import pytest
import torch

from ejkernel_amd.workloads import Batch, make_batch, make_workload
from oracle import rpa_oracle as O
from tests.helpers import oracle_args, run_exact, run_strict, to_np


def _batch(q_lens, kv_lens, **kw):
    args = dict(num_q_heads=4, num_kv_heads=2, head_dim=16, page_size=4, pages_per_seq=8, seed=3,
                dtype=torch.float32)
    args.update(kw)
    return make_batch(q_lens, kv_lens, **args)


def _coded_v(batch):
    """Overwrite V with a value that names (page, slot, kv head, d) exactly in fp32/bf16-free form."""
    P, page, H2, D = batch.kv_pages.shape
    pg = torch.arange(P).view(P, 1, 1, 1).float()
    sl = torch.arange(page).view(1, page, 1, 1).float()
    hd = torch.arange(H2 // 2).view(1, 1, H2 // 2, 1).float()
    dd = torch.arange(D).view(1, 1, 1, D).float()
    code = pg * 64.0 + sl * 4.0 + hd + dd / 64.0  # distinct, exactly representable in fp32
    batch.kv_pages[:, :, 1::2, :] = code
    return code


# ----------------------------------------------------------------------------- bf16 helpers


def test_bf16_round_matches_torch():
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 10,
                        np.float32([0.0, -0.0, 1.0, 1.00390625, 1.01171875, np.inf, -np.inf, 3.3895314e38, 1e-40])])
    want = torch.from_numpy(x).to(torch.bfloat16).to(torch.float32).numpy()
    got = O.bf16_round(x)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert np.isnan(O.bf16_round(np.float32([np.nan]))[0])
    assert np.array_equal(O.bf16_from_bits(O.bf16_bits(got)), got)


# ----------------------------------------------------------------------------- closed forms


@pytest.mark.parametrize("fn", ["exact", "strict"])
def test_zero_query_gives_mean_of_visible_values(fn):
    """q = 0 => all visible logits equal => out = mean of visible V rows (gather, de-interleave, GQA map)."""
    b = _batch([3, 1, 5], [9, 14, 5], pages_per_seq=4, num_pages=40)
    b.queries.zero_()
    code = _coded_v(b)
    out = run_exact(b) if fn == "exact" else run_strict(b, compute_dtype="float32")
    bt = to_np(b.block_tables)
    cu = to_np(b.query_start_loc)
    G = 2
    for s in range(3):
        for i in range(int(b.q_lens[s])):
            pos = int(b.kv_lens[s] - b.q_lens[s]) + i
            for h in range(4):
                rows = [code[bt[s, k // 4], k % 4, h // G, :].numpy() for k in range(pos + 1)]
                want = np.mean(np.asarray(rows, np.float64), axis=0)
                np.testing.assert_allclose(out[cu[s] + i, h], want, rtol=2e-6, atol=1e-5)


@pytest.mark.parametrize("fn", ["exact", "strict"])
def test_single_key_returns_its_value_row(fn):
    b = _batch([1, 1], [1, 1], pages_per_seq=2)
    out = run_exact(b) if fn == "exact" else run_strict(b, compute_dtype="float32")
    kv = to_np(b.kv_pages)
    bt = to_np(b.block_tables)
    for s in range(2):
        for h in range(4):
            np.testing.assert_allclose(out[s, h], kv[bt[s, 0], 0, 2 * (h // 2) + 1], rtol=0, atol=1e-6)


def test_window_bounds_via_position_average():
    """q = 0 and V = key position => out = mean position of the visible keys = (lo + hi - 1) / 2."""
    W = 5
    b = _batch([4], [19], pages_per_seq=8, sliding_window=W)
    b.queries.zero_()
    bt = to_np(b.block_tables)
    for k in range(19):
        b.kv_pages[bt[0, k // 4], k % 4, 1::2, :] = float(k)
    for out in (run_exact(b), run_strict(b, compute_dtype="float32")):
        for i in range(4):
            pos = 15 + i
            lo, hi = max(0, pos - W + 1), pos + 1
            assert hi - lo == min(pos + 1, W)
            np.testing.assert_allclose(out[i], (lo + hi - 1) / 2.0, rtol=1e-6)


def test_two_key_soft_cap_closed_form():
    cap = 1.5
    b = _batch([1], [2], num_q_heads=1, num_kv_heads=1, head_dim=4, pages_per_seq=1, logits_soft_cap=cap,
               softmax_scale=0.7)
    q = to_np(b.queries)[0, 0].astype(np.float64)
    kv = to_np(b.kv_pages).astype(np.float64)
    pg = int(b.block_tables[0, 0])
    k0, v0, k1, v1 = kv[pg, 0, 0], kv[pg, 0, 1], kv[pg, 1, 0], kv[pg, 1, 1]
    l0 = cap * math.tanh(0.7 * float(q @ k0) / cap)
    l1 = cap * math.tanh(0.7 * float(q @ k1) / cap)
    w0 = 1.0 / (1.0 + math.exp(l1 - l0))
    want = w0 * v0 + (1 - w0) * v1
    np.testing.assert_allclose(run_exact(b)[0, 0], want, rtol=1e-12)
    np.testing.assert_allclose(run_strict(b, compute_dtype="float32")[0, 0], want, rtol=2e-6, atol=2e-6)


def test_cap_that_bf16_does_not_hold_is_rounded_before_use():
    """The cap is a weakly typed scalar: in a bf16 program it is 23.75, not 23.7 (closed form worked out by hand in
    two_key_cap_batch; with 23.7 the output would be 0.6796875)."""
    from tests.helpers import two_key_cap_batch

    b, want = two_key_cap_batch()
    assert np.all(run_strict(b)[0, 0] == np.float32(want))
    assert np.all(_c_strict(b)[0, 0] == np.float32(want))
    assert abs(run_exact(b)[0, 0, 0] - 8 / (1 + math.exp(23.7 * (math.tanh(20 / 23.7) - math.tanh(16 / 23.7))))) < 1e-12


def test_one_key_one_sink_closed_form():
    b = _batch([1], [1], num_q_heads=2, num_kv_heads=1, head_dim=4, pages_per_seq=1, softmax_scale=0.5)
    sink = np.float32([[0.3], [-1.2]])  # per q head
    q = to_np(b.queries).astype(np.float64)
    kv = to_np(b.kv_pages).astype(np.float64)
    pg = int(b.block_tables[0, 0])
    for name, out in (("exact", run_exact(b, softmax_aux=sink)),
                      ("strict", run_strict(b, compute_dtype="float32", softmax_aux=sink))):
        for h in range(2):
            s = 0.5 * float(q[0, h] @ kv[pg, 0, 0])
            w = math.exp(s) / (math.exp(s) + math.exp(float(sink[h, 0])))
            np.testing.assert_allclose(out[0, h], w * kv[pg, 0, 1], rtol=3e-6, atol=1e-6, err_msg=name)


def _one_key_one_sink_bf16(sink):
    """One bf16 decode row over one key with logit 0.5 exactly, and V values across five binades."""
    b = _batch([1], [1], num_q_heads=1, num_kv_heads=1, head_dim=8, pages_per_seq=1, softmax_scale=1.0,
               dtype=torch.bfloat16)
    pg = int(b.block_tables[0, 0])
    b.queries.zero_()
    b.queries[0, 0, 0] = 1.0
    b.kv_pages.zero_()
    b.kv_pages[pg, 0, 0, 0] = 0.5
    v = torch.tensor([1.0, 3.0, 100.0, -7.5, 0.4375, 21.0, -1.25, 13.0])
    b.kv_pages[pg, 0, 1] = v.to(torch.bfloat16)
    return b, v.double().numpy(), np.float32([[sink]])


def test_float32_sinks_promote_the_epilogue_of_a_bf16_carry():
    """The reference keeps `softmax_aux` in its own dtype (_xla_impl_fwd.py:60-77), so with float32 sinks and a bf16
    carry `jnp.maximum(max_block, s_max)` (:166) is float32 and everything after it too, with one cast at the end
    (:179): the result is the float64 closed form rounded to bf16 once.  With sinks as narrow as the carry every op
    of :166-172 rounds to bf16, which here lands 1.3 % away: sink 5.3 becomes 5.3125, exp(-4.8125) and 1 + that
    round again.  A restatement that rounds the epilogue whatever the sinks' dtype fails the first half."""
    b, v, sink = _one_key_one_sink_bf16(5.3)
    w = math.exp(0.5) / (math.exp(0.5) + math.exp(float(np.float32(5.3))))
    want = w * v
    rounded = O.bf16_round(want.astype(np.float32)).astype(np.float64)
    step = 2.0 ** (np.floor(np.log2(np.abs(want))) - 7)
    # the closed form is not within float32 noise of a rounding boundary, so one final cast decides the result
    assert (np.abs(np.abs(want - rounded) - step / 2) > 1e-4 * step).all()
    wide = run_strict(b, softmax_aux=sink, aux_dtype="float32")[0, 0].astype(np.float64)
    np.testing.assert_array_equal(wide, rounded)
    # by hand, every op rounded to bf16: m_tot = 5.3125, e_m = bf16(exp(-4.8125)) = 133 * 2**-14,
    # denom = bf16(e_m * 1 + 1) = 1.0078125, out = bf16(bf16(e_m * v) / denom)
    e_m, denom = 133 * 2.0 ** -14, 1.0078125
    assert O.bf16_round(np.float32([math.exp(-4.8125)]))[0] == e_m and O.bf16_round(np.float32([e_m + 1]))[0] == denom
    by_hand = O.bf16_round((O.bf16_round((e_m * v).astype(np.float32)).astype(np.float64) / denom).astype(np.float32))
    narrow = run_strict(b, softmax_aux=sink, aux_dtype="bfloat16")[0, 0].astype(np.float64)
    np.testing.assert_array_equal(narrow, by_hand.astype(np.float64))
    assert (np.abs(narrow - wide) >= step).all(), (narrow, wide)  # the two epilogues are at least one bf16 step apart
    # float32 storage has one epilogue whatever the sinks' dtype says
    b32, _, _ = _one_key_one_sink_bf16(5.3)
    b32.queries, b32.kv_pages = b32.queries.float(), b32.kv_pages.float()
    np.testing.assert_allclose(run_strict(b32, softmax_aux=sink)[0, 0], want, rtol=3e-6)


@pytest.mark.parametrize("aux_dtype", ["float32", "bfloat16"])
def test_c_restatement_follows_the_sinks_dtype(aux_dtype):
    from oracle.rpa_oracle_c import rpa_strict_c

    b, _, sink = _one_key_one_sink_bf16(5.3)
    got = rpa_strict_c(*oracle_args(b), softmax_scale=1.0, softmax_aux=sink, io_dtype="bfloat16", threads=1,
                       aux_dtype=aux_dtype)
    np.testing.assert_array_equal(got[0], run_strict(b, softmax_aux=sink, aux_dtype=aux_dtype)[0])
    rng = np.random.default_rng(5)
    b = make_batch([5, 1, 12], [300, 1000, 12], num_q_heads=4, num_kv_heads=2, head_dim=64, page_size=8,
                   pages_per_seq=128, seed=12, dtype=torch.bfloat16)
    aux = (3.0 * rng.standard_normal((4, 3))).astype(np.float32)
    if aux_dtype == "bfloat16":
        aux = O.bf16_round(aux)
    got = rpa_strict_c(*oracle_args(b), softmax_scale=b.softmax_scale, softmax_aux=aux, io_dtype="bfloat16", threads=2,
                       aux_dtype=aux_dtype)
    want = run_strict(b, softmax_aux=aux, aux_dtype=aux_dtype)
    d = np.abs(got - want)[: b.total_valid_tokens]
    assert d.max() <= 8e-3 and (d > 0).mean() < 2e-3, (d.max(), (d > 0).mean())


# ----------------------------------------------------------------------------- invariants


def test_page_permutation_invariance():
    b = _batch([2, 1, 6], [13, 30, 6], pages_per_seq=8)
    base_e, base_s = run_exact(b), run_strict(b, compute_dtype="float32")
    P = b.kv_pages.shape[0]
    perm = torch.from_numpy(np.random.default_rng(5).permutation(P))
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(P)
    b2 = Batch(**{**b.__dict__})
    b2.kv_pages = b.kv_pages[perm]           # new page i holds old page perm[i]
    b2.block_tables = inv[b.block_tables.long()].to(torch.int32)
    assert np.array_equal(run_exact(b2), base_e)
    assert np.array_equal(run_strict(b2, compute_dtype="float32"), base_s)


def test_window_at_least_kv_len_is_no_window():
    b = _batch([3, 1], [17, 32], pages_per_seq=8)
    base = run_exact(b)
    b.sliding_window = 32
    np.testing.assert_allclose(run_exact(b), base, rtol=0, atol=0)
    b.sliding_window = 31  # now the decode row of sequence 1 loses key 0
    assert np.abs(run_exact(b)[3] - base[3]).max() > 1e-6
    assert np.array_equal(run_exact(b)[:3], base[:3])


def test_huge_cap_is_no_cap():
    b = _batch([3, 1], [17, 32], pages_per_seq=8)
    base = run_exact(b)
    b.logits_soft_cap = 1e9
    np.testing.assert_allclose(run_exact(b), base, rtol=1e-9, atol=1e-12)
    b.logits_soft_cap = 0.5
    assert np.abs(run_exact(b) - base).max() > 1e-3


def test_neg_inf_sink_is_no_sink():
    b = _batch([3, 1], [17, 32], pages_per_seq=8)
    base_e, base_s = run_exact(b), run_strict(b, compute_dtype="float32")
    sink = np.full((2, 3), -np.inf, np.float32)
    np.testing.assert_allclose(run_exact(b, softmax_aux=sink), base_e, rtol=0, atol=0)
    np.testing.assert_allclose(run_strict(b, compute_dtype="float32", softmax_aux=sink), base_s, rtol=0, atol=1e-7)
    sink[:] = 2.0
    assert np.abs(run_exact(b, softmax_aux=sink) - base_e).max() > 1e-3


def test_sink_shapes_are_equivalent():
    b = _batch([2], [11], pages_per_seq=4)
    per_kv = np.float32([[0.1, -0.4], [0.7, 0.2]])
    per_q = np.repeat(per_kv, 2, axis=0)
    a = run_exact(b, softmax_aux=per_kv)
    assert np.array_equal(a, run_exact(b, softmax_aux=per_q))
    shared = np.float32([0.1, -0.4])
    c = run_exact(b, softmax_aux=shared)
    assert np.array_equal(c[:, :2], a[:, :2])  # kv head 0 has exactly these sinks


def test_batch_composition_invariance():
    """Rows of a sequence do not depend on the other sequences, their order, or padding entries."""
    b = _batch([2, 0, 1, 5], [13, 7, 30, 9], pages_per_seq=8, max_num_seqs=6)
    full = run_exact(b)
    cu = to_np(b.query_start_loc)
    for s in (0, 2, 3):
        from ejkernel_amd.workloads import compact_for_host
        sub = compact_for_host(b, [s])
        alone = run_exact(sub)
        n = int(b.q_lens[s])
        np.testing.assert_allclose(alone[:n], full[cu[s]:cu[s] + n], rtol=0, atol=0)
    assert not full[int(cu[4]):].any()  # rows beyond the batch stay zero


def test_rows_beyond_kv_entries_are_never_read():
    """Block-table entries past ceil(kv_len / page) may hold garbage; the exact oracle must not touch them."""
    b = _batch([1, 2], [5, 10], pages_per_seq=8)
    base = run_exact(b)
    bt = b.block_tables.clone()
    bt[0, 2:] = -7
    bt[1, 3:] = 10**6
    b.block_tables = bt
    assert np.array_equal(run_exact(b), base)


# ----------------------------------------------------------------------------- library routine


@pytest.mark.parametrize("q_len,kv_len", [(7, 7), (3, 20), (1, 33)])
def test_contiguous_case_is_textbook_sdpa(q_len, kv_len):
    """Identity block table + one sequence == softmax(scale QK^T + causal mask) V with KV heads repeated."""
    b = _batch([q_len], [kv_len], num_q_heads=6, num_kv_heads=2, head_dim=8, page_size=4, pages_per_seq=9,
               permute_pages=False)
    kv = b.kv_pages.double().reshape(-1, 4, 8)[:kv_len]  # [kv, 2*Hkv, D]
    k = kv[:, 0::2].repeat_interleave(3, dim=1).permute(1, 0, 2)  # [Hq, kv, D]
    v = kv[:, 1::2].repeat_interleave(3, dim=1).permute(1, 0, 2)
    q = b.queries[:q_len].double().permute(1, 0, 2)
    pos = (kv_len - q_len) + torch.arange(q_len)
    mask = torch.arange(kv_len)[None, :] <= pos[:, None]
    want = torch.nn.functional.scaled_dot_product_attention(q, k, v, attn_mask=mask, scale=b.softmax_scale)
    want = want.permute(1, 0, 2).numpy()
    np.testing.assert_allclose(run_exact(b)[:q_len], want, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(run_strict(b, compute_dtype="float32")[:q_len], want, rtol=2e-5, atol=2e-6)


# ----------------------------------------------------------------------------- brute force


def _brute(q, kv, ctx, bt, cu, nseq, scale, cap, window, sinks):
    T, Hq, D = q.shape
    page = kv.shape[1]
    Hkv = kv.shape[2] // 2
    G = Hq // Hkv
    out = np.zeros((T, Hq, D))
    for s in range(nseq):
        ql, kl = cu[s + 1] - cu[s], ctx[s]
        for i in range(ql):
            pos = kl - ql + i
            for h in range(Hq):
                j = h // G
                logits, vals = [], []
                for k in range(kl):
                    if k > pos or (window is not None and k <= pos - window):
                        continue
                    krow = kv[bt[s, k // page], k % page, 2 * j]
                    x = scale * sum(float(q[cu[s] + i, h, d]) * float(krow[d]) for d in range(D))
                    if cap is not None:
                        x = cap * math.tanh(x / cap)
                    logits.append(x)
                    vals.append(kv[bt[s, k // page], k % page, 2 * j + 1].astype(np.float64))
                extra = [] if sinks is None else [float(z) for z in sinks[h]]
                m = max(logits + extra)
                w = [math.exp(x - m) for x in logits]
                den = sum(w) + sum(math.exp(z - m) for z in extra)
                out[cu[s] + i, h] = sum(wi * vi for wi, vi in zip(w, vals)) / den
    return out


@pytest.mark.parametrize("seed", range(6))
def test_brute_force_on_tiny_ragged_batches(seed):
    rng = np.random.default_rng(100 + seed)
    page = int(rng.choice([1, 2, 4]))
    D = int(rng.choice([4, 8]))
    Hkv = int(rng.choice([1, 2]))
    G = int(rng.choice([1, 2, 3]))
    S = int(rng.integers(1, 5))
    pps = int(rng.integers(3, 7))
    kv_lens = rng.integers(1, pps * page + 1, size=S)
    q_lens = np.array([rng.integers(0, min(k, 5) + 1) for k in kv_lens])
    window = None if seed % 2 == 0 else int(rng.integers(1, 6))
    cap = None if seed % 3 == 0 else float(rng.uniform(0.5, 3.0))
    sinks = None if seed % 2 == 1 else rng.standard_normal((Hkv * G, 2)).astype(np.float32)
    b = make_batch(q_lens, kv_lens, num_q_heads=Hkv * G, num_kv_heads=Hkv, head_dim=D, page_size=page,
                   pages_per_seq=pps, seed=seed, dtype=torch.float32, max_num_seqs=S + 1, sliding_window=window,
                   logits_soft_cap=cap)
    bt = b.block_tables.clone()
    for s in range(S):  # garbage beyond the pages in use
        bt[s, -(-int(kv_lens[s]) // page):] = -1
    b.block_tables = bt
    q, kv, ctx, bt_np, cu, ns = oracle_args(b)
    want = _brute(q, kv, ctx, bt_np, cu, int(ns[0]), b.softmax_scale, cap, window, sinks)
    np.testing.assert_allclose(run_exact(b, softmax_aux=sinks), want, rtol=1e-9, atol=1e-12)


# ----------------------------------------------------------------------------- strict vs exact


def test_strict_fp32_tracks_exact_on_ragged_batch():
    b = _batch([9, 1, 0, 17, 2], [40, 64, 8, 17, 33], num_q_heads=8, num_kv_heads=2, head_dim=32, page_size=8,
               pages_per_seq=8, sliding_window=None)
    rows = b.total_valid_tokens
    d = np.abs(run_strict(b, compute_dtype="float32")[:rows] - run_exact(b)[:rows])
    assert d.max() < 1e-5


def test_strict_bf16_tracks_exact_within_tolerance():
    b = make_workload("decode_small")
    rows = b.total_valid_tokens
    s, e = run_strict(b), run_exact(b)
    d = np.abs(s[:rows] - e[:rows])
    assert d.max() <= 2e-2 and d.mean() <= 2e-3
    assert np.array_equal(O.bf16_round(s), s)  # outputs are bf16 values


def test_strict_block_structure_with_cap_window_and_many_kv_blocks():
    """pages_per_seq = 128 gives two 64-page KV blocks: exercises the bf16 carry rescale."""
    b = make_batch([5, 1], [500, 1000], num_q_heads=4, num_kv_heads=2, head_dim=64, page_size=8, pages_per_seq=128,
                   seed=11, logits_soft_cap=30.0)
    rows = b.total_valid_tokens
    d = np.abs(run_strict(b)[:rows] - run_exact(b)[:rows])
    assert d.max() <= 2e-2 and d.mean() <= 2e-3


# ----------------------------------------------------------------------------- documented defects of the reference


def test_strict_reproduces_query_block_clamp_without_slack_rows():
    """Without slack rows the 8-row window of every decode sequence clamps onto rows 0..7: only the last row is right."""
    b = make_batch(np.ones(8, int), [20, 31, 9, 17, 25, 12, 30, 16], num_q_heads=4, num_kv_heads=2, head_dim=16,
                   page_size=4, pages_per_seq=8, seed=2, dtype=torch.float32, slack_rows=0)
    assert b.queries.shape[0] == 8
    strict, exact = run_strict(b, compute_dtype="float32"), run_exact(b)
    assert np.abs(strict[7] - exact[7]).max() < 1e-5
    assert np.abs(strict[:7] - exact[:7]).max() > 1e-2
    b2 = make_batch(np.ones(8, int), [20, 31, 9, 17, 25, 12, 30, 16], num_q_heads=4, num_kv_heads=2, head_dim=16,
                    page_size=4, pages_per_seq=8, seed=2, dtype=torch.float32)
    assert np.abs(run_strict(b2, compute_dtype="float32")[:8] - run_exact(b2)[:8]).max() < 1e-5


def test_strict_reproduces_nan_when_leading_kv_block_is_outside_window():
    b = make_batch([2], [400], num_q_heads=2, num_kv_heads=1, head_dim=16, page_size=4, pages_per_seq=128, seed=4,
                   dtype=torch.float32, sliding_window=50)
    strict = run_strict(b, compute_dtype="float32")  # KV block = 64 pages * 4 = 256 keys, all left of the window
    assert np.isnan(strict[:2]).all()
    assert np.isfinite(run_exact(b)[:2]).all()
    b.sliding_window = 200  # window reaches into the first block: finite again and equal to exact
    assert np.abs(run_strict(b, compute_dtype="float32")[:2] - run_exact(b)[:2]).max() < 1e-5


def test_strict_reproduces_block_table_clamp():
    """pages_per_seq = 96 (>= 64, not a multiple of 64): the second block-table window clamps and misaligns keys."""
    b = make_batch([1], [90 * 4], num_q_heads=2, num_kv_heads=1, head_dim=16, page_size=4, pages_per_seq=96, seed=6,
                   dtype=torch.float32)
    assert np.abs(run_strict(b, compute_dtype="float32")[:1] - run_exact(b)[:1]).max() > 1e-3


# ----------------------------------------------------------------------------- algorithmic counts


def test_algorithmic_counts_small_case():
    c = O.algorithmic_counts([10, 7], [0, 3, 4], [2], num_q_heads=4, num_kv_heads=2, head_dim=8, page_size=4,
                             sliding_window=None)
    pairs = (8 + 9 + 10) + 7
    assert c["pairs"] == pairs and c["flops"] == 4 * 8 * 4 * pairs
    assert c["kv_bytes"] == (10 + 7) * 2 * 2 * 8 * 2 and c["tokens"] == 4
    cw = O.algorithmic_counts([10, 7], [0, 3, 4], [2], num_q_heads=4, num_kv_heads=2, head_dim=8, page_size=4,
                              sliding_window=2)
    assert cw["pairs"] == 2 * 4 and cw["kv_bytes"] == (min(10, 3 + 1) + min(7, 1 + 1)) * 2 * 2 * 8 * 2


# ----------------------------------------------------------------------------- C restatement vs NumPy restatement


def _c_strict(b, softmax_aux=None, threads=2):
    from oracle.rpa_oracle_c import rpa_strict_c

    dt = "bfloat16" if b.queries.dtype == torch.bfloat16 else "float32"
    return rpa_strict_c(*oracle_args(b), softmax_scale=b.softmax_scale, logits_soft_cap=b.logits_soft_cap,
                        sliding_window=b.sliding_window, softmax_aux=softmax_aux, io_dtype=dt, threads=threads)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_c_restatement_matches_numpy_restatement(dtype):
    """Same algorithm, same rounding points: only fp32 summation order may differ (a last-place flip at most)."""
    rng = np.random.default_rng(8)
    sinks = rng.standard_normal((2, 2)).astype(np.float32)
    cases = [
        (make_workload("decode_small", dtype=dtype), None),
        (make_batch([9, 1, 0, 17, 2], [40, 64, 8, 17, 33], num_q_heads=8, num_kv_heads=2, head_dim=32, page_size=8,
                    pages_per_seq=8, seed=1, dtype=dtype, sliding_window=20, logits_soft_cap=5.0, max_num_seqs=7), None),
        (make_batch([5, 1], [500, 1000], num_q_heads=4, num_kv_heads=2, head_dim=64, page_size=8, pages_per_seq=128,
                    seed=11, dtype=dtype), sinks),
    ]
    for b, aux in cases:
        rows = b.total_valid_tokens
        want = run_strict(b, softmax_aux=aux)
        got = _c_strict(b, softmax_aux=aux)
        d = np.abs(got[:rows] - want[:rows])
        if dtype == torch.bfloat16:  # rounded results: identical except where a sum sat on a rounding boundary
            assert d.max() <= 4e-3 and (d > 0).mean() < 2e-3, (d.max(), (d > 0).mean())
        else:
            assert d.max() <= 2e-6, d.max()
        assert not got[rows:].any()


def test_c_restatement_reproduces_window_nan():
    b = make_batch([2], [400], num_q_heads=2, num_kv_heads=1, head_dim=16, page_size=4, pages_per_seq=128, seed=4,
                   dtype=torch.float32, sliding_window=50)
    assert np.isnan(_c_strict(b)[:2]).all()
    b.sliding_window = 200
    assert np.abs(_c_strict(b)[:2] - run_exact(b)[:2]).max() < 1e-5
