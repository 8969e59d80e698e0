"""NumPy restatement of the reference's ``ragged_page_attention_v3`` (cache update + attention).

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

The reference program is ``ejkernel/kernels/_xla/ragged_page_attention_v3/_kernel.py:127-318``
(entry ``_interface.py:25-96``).  Per sequence ``i < distribution[2]``, in order:

1. gather the sequence's pages (``:203-205``), overwrite positions
   ``[kv_len - q_len, kv_len)`` with the new tokens' fused K/V rows (``:207-210``;
   ``merge_kv`` ``:44-57`` puts K of kv head j at combined row 2j and V at 2j + 1)
   and scatter the pages ``< ceil(kv_len / page)`` back (``:212-217``);
2. dense attention over the updated rows in float32 (``:219-262``):
   ``S = (Q / q_scale) K^T * softmax_scale * k_scale * q_scale``, optional
   ``cap * tanh(S / cap)``, ``mask_value`` added where the key is past ``kv_len``,
   in the causal future (``kv_len - q_len + i < k``) or left of the window
   (``kv_len - q_len + i - W >= k``), ``softmax`` in float32, P cast to the cache
   dtype, ``O = P V * v_scale``, rows past ``q_len`` zeroed, cast to the query dtype;
3. the first ``B = min(pages_per_seq * page, T)`` rows of O are written at ``q_start``
   (``:264-291``), so the rows a sequence does not own are zeroed until their owner
   (a later sequence) overwrites them, and rows past the last sequence stay zero.

Two functions:

``rpa_v3_literal``  follows the program step by step with the full
    ``[kv_cap, kv_cap]`` score matrix, the ``mask_value`` addition and the block write.
    Quadratic in ``pages_per_seq * page``: tiny shapes only.
``rpa_v3``          computes the same thing on the visible keys only (a masked entry
    contributes ``exp(S + mask_value - max) == 0`` exactly in float32), usable at
    benchmark sizes.

Arrays are float32 holding values representable in their dtype: ``cache_dtype`` for the cache and
the new keys / values ("bfloat16", "float32", "float8_e4m3fn" or "float8_e5m2"), ``query_dtype`` for the queries
(the cache dtype unless given; "bfloat16" with an 8-bit cache).  The output takes the query dtype
(``:190``), ``Q / q_scale`` is computed in it, clipped to the cache dtype's finite range and cast
to the cache dtype (``:249-254``), and the normalised probabilities are cast to the cache dtype
(``:279``).

Not restated: what XLA does when a block table repeats a page id among the entries the
scatter writes (``.at[indices].set`` with duplicate indices has no defined winner) and
how it clamps or wraps page ids outside the pool; both functions require the pages a
sequence uses to be distinct and in range, and never touch entries past
``ceil(kv_len / page)``.

Parity status: the reference holds no golden vectors for this program and cannot be
imported here (no jax).  Pins (``tests/test_v3_oracle_pins.py``): ``rpa_v3`` against
``rpa_v3_literal`` on random tiny batches; the cache update against a closed form
(every new row lands at its page and slot, nothing else changes); the attention
against the float64 dense oracle of the v2 operation on the updated cache; ``q = 0``
closed form.  For an 8-bit cache: the e4m3 rounding against the cast of torch on 3e5
values including ties and subnormals; closed forms for the cast of the normalised
probabilities (p = 2**-6 survives, p = 2**-10 becomes zero) and for the clip of
``Q / q_scale`` to +-448; ``rpa_v3`` against ``rpa_v3_literal``.  **Parity unpinned:** the
summation order of XLA's float32 matmul / softmax reductions (below 1e-5 relative), and
with an 8-bit cache which side of a rounding boundary a probability falls on when that
order moves it across.
"""

from __future__ import annotations

import numpy as np

from .rpa_oracle import _rounder

DEFAULT_MASK_VALUE = np.float32(-0.7 * float(np.finfo(np.float32).max))  # _kernel.py:25


def packing(cache_dtype):
    """32 // bit width (_kernel.py:38-39)."""
    return {"bfloat16": 2, "float8_e4m3fn": 4, "float8_e5m2": 4}.get(cache_dtype, 1)


def merge_kv(k, v, cache_dtype="bfloat16"):
    """[T, Hkv, D] x 2 -> [T, Hx2 / pack, pack, Dalign] (_kernel.py:44-57)."""
    T, Hkv, D = k.shape
    pack = packing(cache_dtype)
    hx2_act = 2 * Hkv
    hx2 = -(-hx2_act // pack) * pack
    dalign = -(-D // 128) * 128
    kv = np.concatenate([k, v], axis=-1).reshape(T, hx2_act, D)
    kv = np.pad(kv, ((0, 0), (0, hx2 - hx2_act), (0, dalign - D)))
    return kv.reshape(T, hx2 // pack, pack, dalign)


def _unpack(flat, num_kv_heads, dalign):
    """[Tcap, Hx2 / pack, pack, Dalign] -> K, V [Tcap, Hkv, Dalign] (_kernel.py:60-68)."""
    tcap = flat.shape[0]
    kv = flat.reshape(tcap, -1, dalign)[:, : 2 * num_kv_heads, :].reshape(tcap, num_kv_heads, 2 * dalign)
    return kv[:, :, :dalign], kv[:, :, dalign:]


def _clip_to(x, cache_dtype):
    """jnp.clip(x, finfo.min, finfo.max) of the cache dtype (_kernel.py:251-253): only an 8-bit range cuts anything."""
    top = {"float8_e4m3fn": 448.0, "float8_e5m2": 57344.0}.get(cache_dtype)
    return x if top is None else np.clip(x, np.float32(-top), np.float32(top))


def _softmax_f32(s):
    m = s.max(axis=-1, keepdims=True)
    e = np.exp((s - m).astype(np.float32)).astype(np.float32)
    return (e / e.sum(axis=-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def _prep(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution):
    queries = np.asarray(queries, dtype=np.float32)
    keys = np.asarray(keys, dtype=np.float32)
    values = np.asarray(values, dtype=np.float32)
    cache = np.array(kv_cache, dtype=np.float32, copy=True)
    kv_lens = np.asarray(kv_lens).astype(np.int64)
    block_tables = np.asarray(block_tables).astype(np.int64).reshape(-1)
    qsl = np.asarray(query_start_loc).astype(np.int64)
    num_seqs = int(np.asarray(distribution).reshape(-1)[-1])
    max_num_seqs = kv_lens.shape[0]
    assert block_tables.size % max_num_seqs == 0
    return queries, keys, values, cache, kv_lens, block_tables, qsl, min(max(num_seqs, 0), max_num_seqs)


def rpa_v3_literal(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution, *,
                   softmax_scale=1.0, sliding_window=None, logits_soft_cap=None, q_scale=None, k_scale=None,
                   v_scale=None, cache_dtype="bfloat16", query_dtype=None):
    """Step-by-step restatement (_kernel.py:163-318); returns (out [T, Hq, D], updated cache)."""
    R = _rounder(cache_dtype)
    Rq = _rounder(query_dtype or cache_dtype)
    queries, keys, values, cache, kv_lens, bt, qsl, num_seqs = _prep(
        queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution)
    T, Hq, D = queries.shape
    Hkv = keys.shape[1]
    hrep = Hq // Hkv
    _, page, _, _, dalign = cache.shape
    pps = bt.size // kv_lens.shape[0]
    kv_cap = pps * page
    positions = np.arange(kv_cap)
    B = min(kv_cap, T)
    fused = merge_kv(keys, values, cache_dtype)
    out = np.zeros_like(queries)
    for s in range(num_seqs):
        q_start, q_len, kv_len = int(qsl[s]), int(qsl[s + 1] - qsl[s]), int(kv_lens[s])
        idx = bt[s * pps:(s + 1) * pps]
        page_cnt = -(-kv_len // page)
        used = idx[:page_cnt]
        assert len(set(used.tolist())) == len(used) and used.min(initial=0) >= 0 and used.max(initial=0) < cache.shape[0]
        gathered = cache[np.clip(idx, 0, cache.shape[0] - 1)]  # [pps, page, ...]
        flat = gathered.reshape(kv_cap, *gathered.shape[2:])
        tail = (positions >= kv_len - q_len) & (positions < kv_len)
        src = q_start + (positions - (kv_len - q_len))
        rows = np.where(((src >= 0) & (src < T))[:, None, None, None], fused[np.clip(src, 0, T - 1)], 0.0)
        flat_upd = np.where(tail[:, None, None, None], rows, flat).astype(np.float32)
        upd_pages = flat_upd.reshape(gathered.shape)
        for pg in range(min(page_cnt, pps)):  # pages at or past page_cnt are written back unchanged
            cache[idx[pg]] = upd_pages[pg]
        K, V = _unpack(flat_upd, Hkv, dalign)
        K, V = K[:, :, :D], V[:, :, :D]
        K = np.repeat(K, hrep, axis=1)
        V = np.repeat(V, hrep, axis=1)
        iq = q_start + positions
        Q = np.where((iq < T)[:, None, None], queries[np.clip(iq, 0, T - 1)], 0.0).astype(np.float32)
        if q_scale is not None:
            Q = R(_clip_to(Rq(Q / np.float32(q_scale)), cache_dtype))  # divided in the query dtype, clipped, cast to K's dtype
        S = np.einsum("qhd,khd->hqk", Q, K, dtype=np.float32) * np.float32(softmax_scale)
        if k_scale is not None:
            S = S * np.float32(k_scale)
        if q_scale is not None:
            S = S * np.float32(q_scale)
        q_span = (kv_len - q_len) + positions
        bad = ~(positions < q_len)[:, None] | ~(positions < kv_len)[None, :] | (q_span[:, None] < positions[None, :])
        if sliding_window is not None:
            bad |= (q_span[:, None] - sliding_window) >= positions[None, :]
        if logits_soft_cap is not None:
            S = np.float32(logits_soft_cap) * np.tanh(S / np.float32(logits_soft_cap))
        S = np.where(bad[None], S + DEFAULT_MASK_VALUE, S).astype(np.float32)
        P = R(_softmax_f32(S))
        O = np.einsum("hqk,khd->qhd", P, V, dtype=np.float32)
        if v_scale is not None:
            O = O * np.float32(v_scale)
        O = O * (positions < q_len).astype(np.float32)[:, None, None]
        blk = Rq(O[:B])
        if q_start + B <= T:
            out[q_start:q_start + B] = blk
        else:  # scatter-add of the rows that fit (_kernel.py:273-289); the rows it adds to are still zero or are rewritten
            n = T - q_start
            out[q_start:] = Rq(out[q_start:] + blk[:n])
    return out, cache


def rpa_v3(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution, *,
           softmax_scale=1.0, sliding_window=None, logits_soft_cap=None, q_scale=None, k_scale=None, v_scale=None,
           cache_dtype="bfloat16", query_dtype=None, seqs=None, slack=None):
    """Same results as ``rpa_v3_literal`` from the visible keys only; returns (out, updated cache).

    ``seqs`` restricts the attention (not the cache update) to some sequences; the other rows stay zero.
    ``slack`` (a float array [T, Hq], filled in place) receives, per output row, how far an evaluation of the same
    program with another float32 exponential or summation order may land from this one because of the cast of the
    probabilities to an 8-bit cache type: the sum, over the probabilities that lie within 1e-5 (relative) of a
    rounding boundary of that type, of the rounding step there times the largest |V| of that key.  It is zero for
    almost every row; a checker adds it to its bound.
    """
    R = _rounder(cache_dtype)
    Rq = _rounder(query_dtype or cache_dtype)
    queries, keys, values, cache, kv_lens, bt, qsl, num_seqs = _prep(
        queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution)
    T, Hq, D = queries.shape
    Hkv = keys.shape[1]
    hrep = Hq // Hkv
    P_, page, _, _, dalign = cache.shape
    pps = bt.size // kv_lens.shape[0]
    cache_rows = cache.reshape(P_, page, -1, dalign)  # [P, page, Hx2, Dalign] view: K of head j at 2j, V at 2j + 1
    out = np.zeros_like(queries)
    # 1. cache update, sequence by sequence
    for s in range(num_seqs):
        q_start, q_len, kv_len = int(qsl[s]), int(qsl[s + 1] - qsl[s]), int(kv_lens[s])
        for t in range(q_len):
            pos = kv_len - q_len + t
            if pos < 0 or pos >= min(kv_len, pps * page):
                continue
            pg = int(bt[s * pps + pos // page])
            cache_rows[pg, pos % page] = 0.0  # merge_kv's padding (row tails, combined heads past 2 Hkv) is scattered too
            cache_rows[pg, pos % page, 0:2 * Hkv:2, :D] = keys[q_start + t]
            cache_rows[pg, pos % page, 1:2 * Hkv:2, :D] = values[q_start + t]
    # 2. attention on the updated cache
    for s in (range(num_seqs) if seqs is None else seqs):
        q_start, q_len, kv_len = int(qsl[s]), int(qsl[s + 1] - qsl[s]), int(kv_lens[s])
        if q_len <= 0:
            continue
        n_pages = -(-kv_len // page)
        rows = cache_rows[bt[s * pps:s * pps + n_pages]].reshape(n_pages * page, -1, dalign)[:kv_len]
        K = rows[:, 0:2 * Hkv:2, :D]  # [kv_len, Hkv, D]
        V = rows[:, 1:2 * Hkv:2, :D]
        Q = queries[q_start:q_start + q_len]
        if q_scale is not None:
            Q = R(_clip_to(Rq(Q / np.float32(q_scale)), cache_dtype))
        Qg = Q.reshape(q_len, Hkv, hrep, D)
        S = np.einsum("qjgd,kjd->jgqk", Qg, K, dtype=np.float32, optimize=True) * np.float32(softmax_scale)
        if k_scale is not None:
            S = S * np.float32(k_scale)
        if q_scale is not None:
            S = S * np.float32(q_scale)
        kpos = np.arange(kv_len)
        q_span = (kv_len - q_len) + np.arange(q_len)
        bad = q_span[:, None] < kpos[None, :]
        if sliding_window is not None:
            bad |= (q_span[:, None] - sliding_window) >= kpos[None, :]
        if logits_soft_cap is not None:
            S = np.float32(logits_soft_cap) * np.tanh(S / np.float32(logits_soft_cap))
        S = np.where(bad[None, None], S + DEFAULT_MASK_VALUE, S).astype(np.float32)
        P32 = _softmax_f32(S)
        Pm = R(P32)
        O = np.einsum("jgqk,kjd->qjgd", Pm, V, dtype=np.float32, optimize=True).reshape(q_len, Hq, D)
        if v_scale is not None:
            O = O * np.float32(v_scale)
        out[q_start:q_start + q_len] = Rq(O)
        if slack is not None:
            jump = np.abs(R(P32 * np.float32(1 + 1e-5)) - R(P32 * np.float32(1 - 1e-5)))    # [Hkv, hrep, q, k]
            vmax = np.abs(V.astype(np.float32)).max(axis=2)                                 # [k, Hkv]
            row = np.einsum("jgqk,kj->qjg", jump, vmax).reshape(q_len, Hq)
            slack[q_start:q_start + q_len] = row * np.float32(1.0 if v_scale is None else v_scale)
    return out, cache
