"""NumPy restatement of the reference's ragged paged attention forward.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

Two functions:

``rpa_strict``
    Follows ``ejkernel/kernels/_xla/ragged_page_attention/_xla_impl_fwd.py:39-201``
    operation by operation: 8-row query blocks (``:47``), KV blocks of
    ``min(64, pages_per_seq)`` pages (``:48``), the page gather with K at even and
    V at odd combined-head index (``:113-114``), the masked online softmax with
    the carry ``(o, l, m)`` held in ``compute_dtype`` (``:138-155``), the
    ``1e-6`` clamp of the denominator (``:174``) and the sinks epilogue
    (``:161-172``).  XLA rounds every op's result to the op's dtype, so with
    ``compute_dtype = bfloat16`` each intermediate is rounded to bf16 here too
    (round-to-nearest-even, fp32 arithmetic inside an op).  ``lax.dynamic_slice``
    / ``dynamic_update_slice`` clamp their start index so the window fits
    (``:88-92,106-110,181-185``); that clamping is restated as well, including
    the cases where it corrupts results (no slack rows in ``queries``;
    ``pages_per_seq`` >= 64 and not a multiple of 64).  A row whose first KV
    block is entirely masked by a sliding window turns NaN exactly as in the
    reference (``exp(-inf - -inf)``, ``:146``).

``rpa_exact``
    The intended semantics as a dense masked softmax per sequence in float64,
    following the pure-JAX spec
    ``ejkernel/kernels/_pallas/tpu/ragged_page_attention/_pallas_impl_fwd.py:62-121``
    (same mask: ``_pallas_impl_fwd.py:109-113`` == ``_xla_impl_fwd.py:128-136``),
    plus the sinks formula of ``_xla_impl_fwd.py:161-172``.  No rounding anywhere.

Parity status: the reference's own tests hold no golden vectors for the XLA
path, and the reference cannot be imported where this was written (no jax).
Both functions are therefore pinned by closed forms, invariants, a textbook
SDPA on the contiguous special case and brute force on tiny inputs
(``tests/test_oracle_pins.py``).  What stays **parity unpinned**: the exact
bf16 rounding sequence XLA:CPU applies inside ``rpa_strict`` (which ops it
fuses); it matters only below the stated tolerance (2e-2 max / 2e-3 mean).
"""

from __future__ import annotations

import numpy as np

# --------------------------------------------------------------------------- bf16 helpers


def bf16_round(x):
    """Round float32 values to the nearest bfloat16 (ties to even); result stays float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32)
    bias = ((u >> np.uint32(16)) & np.uint32(1)) + np.uint32(0x7FFF)
    r = ((u + bias) & np.uint32(0xFFFF0000)).view(np.float32)
    nan = np.isnan(x)
    if nan.any():
        r = np.where(nan, np.float32(np.nan), r)
    return r


def bf16_bits(x):
    """float32 array holding bf16-representable values -> uint16 bit patterns."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    return (x.view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def bf16_from_bits(b):
    """uint16 bf16 bit patterns -> float32."""
    b = np.ascontiguousarray(b, dtype=np.uint16)
    return (b.astype(np.uint32) << np.uint32(16)).view(np.float32)


def fp8_e4m3fn_round(a):
    """float32 values rounded to the nearest ``float8_e4m3fn`` (ties to even), as float32.

    OCP e4m3: 4 exponent bits (bias 7), 3 mantissa bits, no infinities; normal numbers from 2**-6 to 448,
    subnormal multiples of 2**-9 below.  A value that rounds past 448 becomes NaN (what the cast does; the
    callers here clip first).
    """
    x = np.asarray(a, dtype=np.float32)
    _, e = np.frexp(x)  # |x| = m 2**e with m in [0.5, 1): the binade's exponent is e - 1
    quantum = np.ldexp(np.float32(1.0), np.maximum(e - 1, -6) - 3).astype(np.float32)
    with np.errstate(invalid="ignore"):
        y = (np.rint(x / quantum) * quantum).astype(np.float32)
    y = np.where(np.abs(y) > np.float32(448.0), np.float32(np.nan), y)
    return np.where(np.isfinite(x), y, np.float32(np.nan)).astype(np.float32)


def fp8_e5m2_round(a):
    """The same for ``float8_e5m2``: 5 exponent bits (bias 15), 2 mantissa bits, normal numbers from 2**-14 to
    57344, subnormal multiples of 2**-16, infinities (a value that rounds past 57344 becomes infinite)."""
    x = np.asarray(a, dtype=np.float32)
    _, e = np.frexp(x)
    quantum = np.ldexp(np.float32(1.0), np.maximum(e - 1, -14) - 2).astype(np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        y = (np.rint(x / quantum) * quantum).astype(np.float32)
    y = np.where(np.abs(y) > np.float32(57344.0), np.copysign(np.float32(np.inf), x), y)
    return np.where(np.isnan(x), np.float32(np.nan), y).astype(np.float32)


def _rounder(dtype):
    name = np.dtype(dtype).name if not isinstance(dtype, str) else dtype
    if name in ("bfloat16", "bf16"):
        return bf16_round
    if name in ("float32", "f32"):
        return lambda a: np.asarray(a, dtype=np.float32)
    if name in ("float8_e4m3fn", "fp8_e4m3"):
        return fp8_e4m3fn_round
    if name in ("float8_e5m2", "fp8_e5m2"):
        return fp8_e5m2_round
    raise ValueError(f"unsupported dtype {dtype!r}")


def _is_f32(dtype):
    name = np.dtype(dtype).name if not isinstance(dtype, str) else dtype
    return name in ("float32", "f32")


def _clamp_start(start, size, total):
    """Start index of a lax.dynamic_slice window of `size` in an axis of length `total`."""
    return int(min(max(int(start), 0), total - size))


def _num_seqs(num_seqs):
    a = np.asarray(num_seqs)
    return int(a.reshape(-1)[0])


def _sinks_per_q_head(softmax_aux, num_q_heads, num_kv_heads):
    """Broadcast sink logits to [num_q_heads, n_sinks] (_xla_impl_fwd.py:60-77)."""
    aux = np.asarray(softmax_aux)
    group = num_q_heads // num_kv_heads
    if aux.ndim == 2:
        if aux.shape[0] == num_q_heads:
            return aux.reshape(num_q_heads, -1)
        if aux.shape[0] == num_kv_heads:
            return np.repeat(aux, group, axis=0)
        raise ValueError(
            f"softmax_aux first dim must be num_q_heads ({num_q_heads}) or num_kv_heads ({num_kv_heads}), "
            f"got {aux.shape}"
        )
    if aux.ndim == 1:
        return np.broadcast_to(aux[None, :], (num_q_heads, aux.shape[0])).copy()
    raise ValueError(f"Unsupported softmax_aux shape: {aux.shape}")


# --------------------------------------------------------------------------- strict restatement


def rpa_strict(
    queries,
    kv_pages,
    context_lens,
    block_tables,
    query_start_loc,
    num_seqs,
    softmax_scale=None,
    logits_soft_cap=None,
    compute_dtype="bfloat16",
    sliding_window=None,
    softmax_aux=None,
    io_dtype="bfloat16",
    aux_dtype="float32",
):
    """Restates ``_ragged_paged_attention`` (_xla_impl_fwd.py:25-201).

    ``queries`` / ``kv_pages`` are float32 arrays whose values are representable in
    ``io_dtype`` (the storage dtype the reference would see).  Returns float32 holding
    ``io_dtype``-representable values, shape ``[T, Hq, D]``.

    ``aux_dtype`` is the dtype the reference would see ``softmax_aux`` in.  The program keeps the sinks in
    that dtype (:60-77), so JAX's promotion decides the precision of the sinks epilogue (:161-172): with
    float32 sinks and a bfloat16 carry, ``jnp.maximum(max_block, s_max)`` is float32 and so is everything
    after it, with the single cast of :179 at the end; with sinks as narrow as the carry every op of the
    epilogue rounds to ``compute_dtype``.  float32 is what the device ABI takes.
    """
    Rq = _rounder(io_dtype)
    Rc = _rounder(compute_dtype)
    # the epilogue's dtype: the wider of the carry's and the sinks' (bf16 with f32 promotes to f32)
    wide_aux = _is_f32(aux_dtype) and not _is_f32(compute_dtype)
    Re = _rounder("float32") if wide_aux else Rc
    Ra = _rounder(aux_dtype)
    queries = np.asarray(queries, dtype=np.float32)
    kv_pages = np.asarray(kv_pages, dtype=np.float32)
    context_lens = np.asarray(context_lens)
    block_tables = np.asarray(block_tables)
    query_start_loc = np.asarray(query_start_loc)

    T, Hq, D = queries.shape
    P, page_size, H2, _ = kv_pages.shape
    Hkv = H2 // 2
    pps = block_tables.shape[-1]
    G = Hq // Hkv
    if softmax_scale is None:  # _interface.py:94-95
        softmax_scale = D**-0.5

    q = queries.reshape(T, Hkv, G, D)
    qblocks = 8 if T >= 8 else max(1, T)  # :47
    kvblocks = 64 if pps >= 64 else max(1, pps)  # :48
    scale_q = Rq(np.float32(softmax_scale))  # weak-typed scalar takes the array's dtype
    q = Rq(q * scale_q)  # :49
    pad = (-T) % qblocks
    if pad:
        q = np.concatenate([q, np.zeros((pad, Hkv, G, D), np.float32)], axis=0)
    Tp = q.shape[0]
    out = np.zeros_like(q)

    sinks = None
    if softmax_aux is not None:
        sinks = _sinks_per_q_head(np.asarray(softmax_aux, np.float32), Hq, Hkv).reshape(Hkv, G, -1)

    kv_tok = page_size * kvblocks
    base_k = np.arange(kv_tok, dtype=np.int64)
    # a Python scalar is weakly typed: XLA converts it to the array's dtype before the op (cap 23.7 is 23.75 in bf16)
    cap = None if logits_soft_cap is None else Rc(np.float32(logits_soft_cap))
    neg_inf = np.float32(-np.inf)

    with np.errstate(invalid="ignore", over="ignore", divide="ignore"):
        for s in range(_num_seqs(num_seqs)):
            q_len = int(query_start_loc[s + 1]) - int(query_start_loc[s])
            if q_len <= 0:  # :189-193
                continue
            kv_len = int(context_lens[s])
            n_qb = (q_len + qblocks - 1) // qblocks
            n_kvb = (kv_len + kv_tok - 1) // kv_tok
            for qb in range(n_qb):
                q_off = qb * qblocks
                g_start = int(query_start_loc[s]) + q_off
                r0 = _clamp_start(g_start, qblocks, Tp)  # dynamic_slice clamp :88-92
                q_blk = Rc(q[r0 : r0 + qblocks])  # [8,Hkv,G,D]
                q_pos = np.arange(qblocks, dtype=np.int64) + (kv_len - q_len + q_off)  # :96-97

                o = np.zeros((qblocks, Hkv, G, D), np.float32)
                l = np.zeros((qblocks, Hkv, G), np.float32)
                m = np.full((qblocks, Hkv, G), neg_inf, np.float32)
                qm = q_blk.transpose(1, 0, 2, 3).reshape(Hkv, qblocks * G, D)

                for kb in range(n_kvb):
                    c0 = _clamp_start(kb * kvblocks, kvblocks, pps)  # :106-110
                    pids = block_tables[s, c0 : c0 + kvblocks].astype(np.int64)
                    pids = np.clip(np.where(pids < 0, pids + P, pids), 0, P - 1)  # gather clamps
                    blk = kv_pages[pids]  # [kvblocks,page,2Hkv,D]
                    k_blk = Rc(blk[:, :, 0::2, :].reshape(kv_tok, Hkv, D))  # :113
                    v_blk = Rc(blk[:, :, 1::2, :].reshape(kv_tok, Hkv, D))  # :114
                    k_ids = base_k + kb * kv_tok

                    sc = np.matmul(qm, k_blk.transpose(1, 2, 0))  # [Hkv, 8G, K]  :119-124
                    sc = Rc(sc).reshape(Hkv, qblocks, G, kv_tok).transpose(1, 0, 2, 3)
                    if cap is not None:  # :125-126
                        sc = Rc(Rc(np.tanh(Rc(sc / cap))) * cap)
                    mask = q_pos[:, None] >= k_ids[None, :]  # :128
                    if sliding_window is not None:  # :129-134
                        mask &= k_ids[None, :] > (q_pos - int(sliding_window))[:, None]
                    mask &= (k_ids < kv_len)[None, :]  # :135
                    mask4 = mask[:, None, None, :]
                    sc = np.where(mask4, sc, neg_inf)  # :138

                    cur = sc.max(axis=3)  # :140
                    new_m = np.maximum(m, cur)  # :141
                    p = Rc(np.exp(Rc(sc - new_m[..., None])))  # :143
                    p = np.where(mask4, p, np.float32(0.0))  # :144
                    resc = Rc(np.exp(Rc(m - new_m)))  # :146  (NaN when both are -inf)
                    psum = Rc(p.sum(axis=3, dtype=np.float32))  # jnp.sum reduces bf16 in fp32
                    l = Rc(Rc(resc * l) + psum)  # :147
                    pm = p.transpose(1, 0, 2, 3).reshape(Hkv, qblocks * G, kv_tok)
                    upd = np.matmul(pm, v_blk.transpose(1, 0, 2))  # [Hkv, 8G, D]  :148
                    upd = Rc(upd).reshape(Hkv, qblocks, G, D).transpose(1, 0, 2, 3)
                    o = Rc(Rc(resc[..., None] * o) + upd)  # :149
                    m = new_m

                if sinks is not None:  # :161-172
                    sb = np.broadcast_to(Ra(sinks)[None], (qblocks, Hkv, G, sinks.shape[-1]))
                    s_max = sb.max(axis=3)
                    m_tot = np.maximum(m, s_max)  # :166, in the promoted dtype
                    e_m = Re(np.exp(Re(m - m_tot)))
                    e_s = Re(np.exp(Re(sb - m_tot[..., None])))
                    denom = Re(Re(e_m * l) + Re(e_s.sum(axis=3, dtype=np.float32)))
                    denom = np.maximum(denom, Re(np.float32(1e-6)))
                    res = Re(Re(e_m[..., None] * o) / denom[..., None])
                else:  # :173-177
                    l = np.maximum(l, Rc(np.float32(1e-6)))
                    res = Rc(o / l[..., None])
                res = Rq(res)  # :179
                out[r0 : r0 + qblocks] = res  # dynamic_update_slice clamps the same way :181-185

    return out[:T].reshape(T, Hq, D)


# --------------------------------------------------------------------------- intended semantics


def visible_range(q_pos, kv_len, sliding_window):
    """[lo, hi) of key positions a query at absolute position ``q_pos`` attends to."""
    hi = min(q_pos + 1, kv_len)
    lo = 0 if sliding_window is None else max(0, q_pos - int(sliding_window) + 1)
    return lo, hi


def rpa_exact(
    queries,
    kv_pages,
    context_lens,
    block_tables,
    query_start_loc,
    num_seqs,
    softmax_scale=None,
    logits_soft_cap=None,
    sliding_window=None,
    softmax_aux=None,
    dtype=np.float64,
    kv_start=None,
):
    """Dense per-sequence evaluation of the intended semantics in ``dtype`` (float64).

    ``kv_start`` (optional, one entry per sequence) drops the keys before that position: the extension of the
    operation that ragged_decode_attention's ``sequence_start`` needs; the reference operation has no such input.

    Follows ``ref_ragged_page_attention`` (_pallas_impl_fwd.py:62-121): gather the
    sequence's pages, split K/V by even/odd combined head, repeat KV heads over the
    query group, ``logits = (q . k) * scale``, optional ``cap * tanh(logits / cap)``,
    mask ``k > q_pos`` or ``k <= q_pos - window``, softmax, ``P @ V``.  Rows at or
    beyond ``query_start_loc[num_seqs]`` are zero.  Only the first
    ``ceil(kv_len / page_size)`` block-table entries of a sequence are read.
    """
    queries = np.asarray(queries, dtype=dtype)
    context_lens = np.asarray(context_lens)
    block_tables = np.asarray(block_tables)
    query_start_loc = np.asarray(query_start_loc)
    T, Hq, D = queries.shape
    P, page_size, H2, _ = kv_pages.shape
    Hkv = H2 // 2
    G = Hq // Hkv
    if softmax_scale is None:
        softmax_scale = D**-0.5
    out = np.zeros((T, Hq, D), dtype=dtype)
    sinks = None
    if softmax_aux is not None:
        sinks = _sinks_per_q_head(np.asarray(softmax_aux, dtype), Hq, Hkv)  # [Hq, n]

    for s in range(_num_seqs(num_seqs)):
        q0, q1 = int(query_start_loc[s]), int(query_start_loc[s + 1])
        q_len = q1 - q0
        if q_len <= 0:
            continue
        kv_len = int(context_lens[s])
        n_pages = (kv_len + page_size - 1) // page_size
        pids = block_tables[s, :n_pages].astype(np.int64)
        blk = np.asarray(kv_pages[pids], dtype=dtype).reshape(n_pages * page_size, H2, D)[:kv_len]
        k = blk[:, 0::2, :]  # [kv, Hkv, D]
        v = blk[:, 1::2, :]
        q = queries[q0:q1].reshape(q_len, Hkv, G, D)
        logits = np.einsum("qjgd,kjd->jgqk", q, k) * dtype(softmax_scale)
        if logits_soft_cap is not None:
            logits = dtype(logits_soft_cap) * np.tanh(logits / dtype(logits_soft_cap))
        q_pos = (kv_len - q_len) + np.arange(q_len)
        k_pos = np.arange(kv_len)
        keep = k_pos[None, :] <= q_pos[:, None]
        if sliding_window is not None:
            keep &= k_pos[None, :] > (q_pos[:, None] - int(sliding_window))
        if kv_start is not None:
            keep &= (k_pos >= int(kv_start[s]))[None, :]
        logits = np.where(keep[None, None], logits, -np.inf)
        m = logits.max(axis=3)  # [j,g,q]
        if sinks is not None:
            sk = sinks.reshape(Hkv, G, -1)  # [j,g,n]
            m = np.maximum(m, sk.max(axis=2)[:, :, None])
        m_safe = np.where(np.isfinite(m), m, 0.0)
        p = np.exp(logits - m_safe[..., None])
        denom = p.sum(axis=3)
        if sinks is not None:
            denom = denom + np.exp(sk[:, :, None, :] - m_safe[..., None]).sum(axis=3)
        denom = np.where(denom > 0, denom, 1.0)
        o = np.einsum("jgqk,kjd->qjgd", p, v) / denom.transpose(2, 0, 1)[..., None]
        out[q0:q1] = o.reshape(q_len, Hq, D)
    return out


# --------------------------------------------------------------------------- algorithmic counts


def algorithmic_counts(context_lens, query_start_loc, num_seqs, num_q_heads, num_kv_heads, head_dim,
                       page_size, sliding_window=None, elem_bytes=2):
    """FLOPs and HBM bytes the workload needs at minimum.

    ``flops = 4 * D * Hq * sum(visible (row, key) pairs)``; every needed K/V token is
    read once per kv head, Q read once, O written once, plus the int32 metadata.
    """
    context_lens = np.asarray(context_lens)
    query_start_loc = np.asarray(query_start_loc)
    S = _num_seqs(num_seqs)
    pairs = 0
    kv_tokens = 0
    pages = 0
    for s in range(S):
        q_len = int(query_start_loc[s + 1]) - int(query_start_loc[s])
        kv_len = int(context_lens[s])
        if q_len <= 0:
            continue
        pos = (kv_len - q_len) + np.arange(q_len, dtype=np.int64)
        vis = pos + 1
        if sliding_window is not None:
            vis = np.minimum(vis, int(sliding_window))
            e = min(kv_len, q_len + int(sliding_window) - 1)
        else:
            e = kv_len
        pairs += int(vis.sum())
        kv_tokens += e
        pages += (e + page_size - 1) // page_size
    t_valid = int(query_start_loc[S])
    flops = 4 * head_dim * num_q_heads * pairs
    kv_bytes = kv_tokens * 2 * num_kv_heads * head_dim * elem_bytes
    qo_bytes = 2 * t_valid * num_q_heads * head_dim * elem_bytes
    meta_bytes = 4 * (pages + 2 * S + 1)
    return dict(flops=flops, kv_bytes=kv_bytes, qo_bytes=qo_bytes, meta_bytes=meta_bytes,
                bytes=kv_bytes + qo_bytes + meta_bytes, tokens=t_valid, pairs=pairs)
