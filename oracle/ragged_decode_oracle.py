"""NumPy restatement of the reference's ``ragged_decode_attention`` (XLA backend), attention sinks included.

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

The reference program is ``ejkernel/kernels/_xla/ragged_decode_attention/_xla_impl_fwd.py``:
``ragged_decode_mqa_xla`` (``:303-364``) runs, per kv head, ``ragged_flash_attention_xla``
(``:201-300``) with one query position: the mask of ``create_attention_mask`` (``:25-82``) --
key ``k`` kept iff ``start <= k < end`` and, with ``sliding_window=(left, right)``,
``end - 1 - left <= k <= end - 1 + right`` -- and a scan over KV blocks of
``fwd_params.kv_blocksize`` keys with ``flash_attention_block`` (``:137-198``), whose carry
``(o, m, l)`` has the query dtype.

``ragged_decode_strict`` follows that scan op by op, rounding each op's result to the query
dtype (``softmax_scale`` is a weakly typed scalar, so nothing is promoted).  It reproduces a
defect of the program: when a sequence's first KV block holds no visible key, ``m_prev - m_new``
is ``-inf - -inf`` and the row turns NaN for good (``:181-183``); this is the case for every
``sequence_start >= kv_blocksize`` and for every window that ends past the first block.
It also reproduces that the scan is not attention once a sequence spans several blocks: the
block's contribution ``o_curr`` is computed from weights already divided by the new normaliser
(``:188-189``) and is then weighted by ``l_curr / l_new`` once more (``:191``), which
under-weights every block after the first.  Only sequences that fit one KV block
(``kv_blocksize >= seq_len``) get attention out of the reference program; the build computes
attention for all of them and is compared with this function on those cases only.
``ragged_decode_exact`` is the dense masked softmax in float64 (zeros when nothing is visible).

Attention sinks (``softmax_aux`` of ``num_sinks`` entries per row).  The program defines them
through the keys: the positions ``[start, start + num_sinks)`` are visible whatever ``end`` and
the window say (``:71-75``; the range is not cut at ``end``), and a key at absolute position
``t < num_sinks`` gets ``softmax_aux[row, t]`` added to its logit after the soft cap and before
the mask (``apply_attention_sinks_block``, ``:98-134``, called at ``:175-176``).  A one-dimensional
``softmax_aux`` serves every head.  A two-dimensional one is added as ``[1, 1, rows, block]`` to
scores of ``[batch, 1, G, block]`` inside the per-kv-head ``vmap`` (``:336-362``; ``softmax_aux``
is closed over, not mapped), so it only broadcasts with ``rows in (1, G)``, ``G`` the query heads
per kv head, and row ``g`` then belongs to the ``g``-th query head of every kv head; any other row
count -- the ``[num_kv_heads, num_sinks]`` of the docstring included, unless it happens to equal
``G`` -- fails to broadcast (``sink_rows`` raises ``ValueError`` for it).  A float32
``softmax_aux`` promotes the biased scores of a bfloat16 call, and with them every later op of
the block, to float32; the carry is cast back at the end of the block (``:198-200``).

Parity status: no golden vectors in the reference, no jax here.  Pins
(``tests/test_ragged_decode_oracle_pins.py``): brute force on tiny inputs, closed forms,
block-size independence of the exact result, agreement with the ragged_page_attention oracle on
the same data viewed as one page per sequence, the NaN defect.  **Parity unpinned:** which bf16
ops XLA:CPU fuses inside the scan body (matters below 2e-2 / 2e-3).
"""

from __future__ import annotations

import numpy as np

from .rpa_oracle import _rounder


def visible(start, end, seq_len, sliding_window, num_sinks=0):
    """create_attention_mask (:25-82) for one sequence and one query position."""
    k = np.arange(seq_len)
    m = (k >= start) & (k < end)
    if sliding_window is not None:
        left, right = sliding_window
        qp = end - 1
        m &= (k >= qp - left) & (k <= qp + right)
    if num_sinks > 0:
        m |= (k >= start) & (k < start + num_sinks)
    return m


def sink_rows(softmax_aux, group):
    """``[G, num_sinks]`` float32 biases as the program broadcasts them (:118-134), or None."""
    if softmax_aux is None:
        return None
    aux = np.asarray(softmax_aux, dtype=np.float32)
    if aux.ndim == 1:
        aux = aux[None, :]
    if aux.ndim != 2 or aux.shape[0] not in (1, group):
        raise ValueError(f"softmax_aux of shape {aux.shape} does not broadcast against {group} query heads per kv head")
    return np.broadcast_to(aux, (group, aux.shape[1]))


def _bias(aux, positions):
    """Bias per (query head of the group, position): softmax_aux[:, t] for t < num_sinks, else 0 (:123-130)."""
    ns = aux.shape[1]
    b = aux[:, np.minimum(positions, ns - 1)]
    return np.where(positions[None, :] < ns, b, np.float32(0.0)).astype(np.float32)


def ragged_decode_strict(query, key, value, sequence_start, sequence_end, softmax_scale=None, block_size=128,
                         sliding_window=None, logits_soft_cap=None, io_dtype="bfloat16", softmax_aux=None,
                         aux_dtype="float32"):
    R = _rounder(io_dtype)  # carries and everything up to the bias
    q = np.asarray(query, dtype=np.float32)
    kk = np.asarray(key, dtype=np.float32)
    vv = np.asarray(value, dtype=np.float32)
    B, Hq, D = q.shape
    _, S, Hkv, _ = kk.shape
    G = Hq // Hkv
    scale = R(np.float32(1.0 / np.sqrt(D) if softmax_scale is None else softmax_scale))
    aux = sink_rows(softmax_aux, G)
    ns = 0 if aux is None else aux.shape[1]
    # ops after the bias run in the promoted dtype
    Rm = R if (aux is None or aux_dtype == io_dtype) else _rounder("float32")
    nblk = -(-S // block_size)
    pad = nblk * block_size - S
    if pad:
        kk = np.pad(kk, ((0, 0), (0, pad), (0, 0), (0, 0)))
        vv = np.pad(vv, ((0, 0), (0, pad), (0, 0), (0, 0)))
    out = np.zeros((B, Hq, D), np.float32)
    with np.errstate(invalid="ignore", over="ignore"):
        for b in range(B):
            mask = np.pad(visible(int(sequence_start[b]), int(sequence_end[b]), S, sliding_window, ns), (0, pad))
            qs = R(q[b].reshape(Hkv, G, D) * scale)
            o = np.zeros((Hkv, G, D), np.float32)
            m = np.full((Hkv, G, 1), -np.inf, np.float32)
            l = np.zeros((Hkv, G, 1), np.float32)
            for i in range(nblk):
                sl = slice(i * block_size, (i + 1) * block_size)
                kb = kk[b, sl].transpose(1, 0, 2)  # [Hkv, bs, D]
                vb = vv[b, sl].transpose(1, 0, 2)
                mb = mask[sl][None, None, :]
                sc = R(np.einsum("jgd,jkd->jgk", qs, kb, dtype=np.float32))
                if logits_soft_cap is not None:
                    cap = R(np.float32(logits_soft_cap))  # weakly typed scalar: the array's dtype first
                    sc = R(R(np.tanh(R(sc / cap))) * cap)
                if aux is not None:
                    sc = Rm(sc + _bias(aux, np.arange(i * block_size, (i + 1) * block_size))[None, :, :])
                sc = np.where(mb, sc, -np.inf).astype(np.float32)
                m_new = np.maximum(m, sc.max(axis=-1, keepdims=True))
                e = Rm(np.exp(Rm(sc - m_new)))
                e = np.where(mb, e, np.float32(0.0))
                l_curr = Rm(e.sum(axis=-1, keepdims=True, dtype=np.float32))
                corr = Rm(np.exp(Rm(m - m_new)))
                l_new = Rm(Rm(corr * l) + l_curr)
                safe = np.where(l_new == 0, np.float32(1.0), l_new)
                w = Rm(e / safe)
                o_curr = Rm(np.einsum("jgk,jkd->jgd", w, vb, dtype=np.float32))
                o = R(Rm(Rm(Rm(Rm(corr * l) * o) + Rm(l_curr * o_curr)) / safe))
                m, l = R(m_new), R(l_new)
            out[b] = o.reshape(Hq, D)
    return out


def ragged_decode_exact(query, key, value, sequence_start, sequence_end, softmax_scale=None, sliding_window=None,
                        logits_soft_cap=None, softmax_aux=None):
    q = np.asarray(query, dtype=np.float64)
    kk = np.asarray(key, dtype=np.float64)
    vv = np.asarray(value, dtype=np.float64)
    B, Hq, D = q.shape
    _, S, Hkv, _ = kk.shape
    G = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if softmax_scale is None else float(softmax_scale)
    aux = sink_rows(softmax_aux, G)
    ns = 0 if aux is None else aux.shape[1]
    out = np.zeros((B, Hq, D))
    for b in range(B):
        vis = visible(int(sequence_start[b]), int(sequence_end[b]), S, sliding_window, ns)
        if not vis.any():
            continue
        k = kk[b, vis].transpose(1, 0, 2)
        v = vv[b, vis].transpose(1, 0, 2)
        sc = np.einsum("jgd,jkd->jgk", q[b].reshape(Hkv, G, D) * scale, k)
        if logits_soft_cap is not None:
            sc = logits_soft_cap * np.tanh(sc / logits_soft_cap)
        if aux is not None:
            sc = sc + _bias(aux, np.flatnonzero(vis)).astype(np.float64)[None, :, :]
        w = np.exp(sc - sc.max(axis=-1, keepdims=True))
        w /= w.sum(axis=-1, keepdims=True)
        out[b] = np.einsum("jgk,jkd->jgd", w, v).reshape(Hq, D)
    return out
