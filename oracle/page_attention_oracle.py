"""NumPy restatement of the reference's ``page_attention`` (XLA backend).

TEST INFRASTRUCTURE ONLY (see ``oracle/__init__.py``).

The reference program is ``ejkernel/kernels/_xla/page_attention/_xla_impl_fwd.py:22-101``
(entry ``_interface.py:25-115``): ``query * attn_scale`` (``:64``); per sequence, for EVERY
entry of its block-table row, ``scores = einsum(q, k_block)`` with positions at or past
``context_len`` replaced by ``-1e9`` (``:76-86``); one ``jax.nn.softmax`` over all
``max_blocks * block_size`` positions (``:94``); ``einsum(weights, values)`` (``:96``).

``page_attention_strict`` rounds after every op to the dtype XLA gives that op:
  * ``attn_scale`` passed as a Python number is weakly typed, so everything stays in the
    query dtype (bf16: ``q * bf16(scale)``, scores, ``x - max``, ``exp``, the sum, the
    quotient and the output are each rounded to bf16);
  * ``attn_scale=None`` makes the scale a float32 array (``_interface.py:110-111``) and
    promotes the computation -- and the result -- to float32.
``page_attention_exact`` is the dense masked softmax in float64.

Out-of-range block ids: JAX wraps negative indices and clamps on gather; both are restated
(``_gather_index``).  A sequence with ``context_len == 0`` softmaxes a row of equal mask
values: the reference returns the mean of whatever its block-table row points at, and so do
these functions.

Parity status: no golden vectors in the reference, no jax here.  Pins
(``tests/test_page_attention_oracle_pins.py``): brute-force loops on tiny inputs, closed
forms (one key; ``q = 0``), block-permutation invariance, and agreement with the separately
written oracle of ragged_page_attention on the same data re-laid-out with one query token per
sequence.  **Parity unpinned:** which of the bf16 ops XLA:CPU fuses (matters below 2e-2 / 2e-3).
"""

from __future__ import annotations

import numpy as np

from .rpa_oracle import _rounder

MASK = -1e9  # _xla_impl_fwd.py:84


def _gather_index(idx, n):
    idx = np.asarray(idx).astype(np.int64)
    idx = np.where(idx < 0, idx + n, idx)
    return np.clip(idx, 0, n - 1)


def page_attention_strict(query, key_cache, value_cache, context_lens, block_tables, attn_scale=None,
                          io_dtype="bfloat16"):
    """Returns float32 [num_seqs, num_heads, head_dim] holding the values of the reference's result dtype."""
    q = np.asarray(query, dtype=np.float32)
    kc = np.asarray(key_cache, dtype=np.float32)
    vc = np.asarray(value_cache, dtype=np.float32)
    S, Hq, D = q.shape
    nb, Hkv, bs, _ = kc.shape
    G = Hq // Hkv
    if attn_scale is None:
        R = _rounder("float32")
        scale = np.float32(1.0) / np.sqrt(np.float32(D))
    else:
        R = _rounder(io_dtype)
        scale = R(np.float32(attn_scale))
    qs = R(q.reshape(S, Hkv, G, D) * scale)
    out = np.zeros((S, Hq, D), np.float32)
    pos = np.arange(np.asarray(block_tables).shape[1] * bs)
    for s in range(S):
        phys = _gather_index(np.asarray(block_tables)[s], nb)
        k = kc[phys].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)  # [Hkv, max_blocks * bs, D]
        v = vc[phys].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)
        sc = R(np.einsum("jgd,jkd->jgk", qs[s], k, dtype=np.float32))
        sc = np.where((pos < int(context_lens[s]))[None, None, :], sc, R(np.float32(MASK)))
        mx = sc.max(axis=-1, keepdims=True)
        un = R(np.exp(R(sc - mx)))
        w = R(un / R(un.sum(axis=-1, keepdims=True, dtype=np.float32)))
        out[s] = R(np.einsum("jgk,jkd->jgd", w, v, dtype=np.float32)).reshape(Hq, D)
    return out


def page_attention_exact(query, key_cache, value_cache, context_lens, block_tables, attn_scale=None):
    """Dense evaluation in float64 over the first ``context_len`` positions (zeros when there are none)."""
    q = np.asarray(query, dtype=np.float64)
    kc = np.asarray(key_cache, dtype=np.float64)
    vc = np.asarray(value_cache, dtype=np.float64)
    S, Hq, D = q.shape
    nb, Hkv, bs, _ = kc.shape
    G = Hq // Hkv
    scale = 1.0 / np.sqrt(D) if attn_scale is None else float(attn_scale)
    out = np.zeros((S, Hq, D))
    for s in range(S):
        n = int(context_lens[s])
        if n <= 0:
            continue
        nblk = -(-n // bs)
        phys = _gather_index(np.asarray(block_tables)[s, :nblk], nb)
        k = kc[phys].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :n]
        v = vc[phys].transpose(1, 0, 2, 3).reshape(Hkv, -1, D)[:, :n]
        sc = np.einsum("jgd,jkd->jgk", q[s].reshape(Hkv, G, D) * scale, k)
        w = np.exp(sc - sc.max(axis=-1, keepdims=True))
        w /= w.sum(axis=-1, keepdims=True)
        out[s] = np.einsum("jgk,jkd->jgd", w, v).reshape(Hq, D)
    return out


def to_interleaved(key_cache, value_cache):
    """[nb, Hkv, bs, D] x 2 -> the [nb, bs, 2 * Hkv, D] layout of ragged_page_attention (K at 2j, V at 2j + 1)."""
    k = np.asarray(key_cache).transpose(0, 2, 1, 3)
    v = np.asarray(value_cache).transpose(0, 2, 1, 3)
    nb, bs, Hkv, D = k.shape
    return np.stack([k, v], axis=3).reshape(nb, bs, 2 * Hkv, D)
