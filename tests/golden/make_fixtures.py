"""Writes the frozen fixtures of this directory: small seeded inputs and the outputs of this repository's CPU oracles.

They are NOT outputs of the reference: ejkernel cannot be imported where this was written (no jax), and its own
tests hold no vectors for these operations.  The fixtures freeze what the oracle restatements computed when they
were pinned (closed forms, brute force, cross-checks: tests/test_*oracle_pins.py), so that a later edit of an
oracle cannot silently change the expected values the device kernels are held to.

    python tests/golden/make_fixtures.py        # rewrites tests/golden/*.npz
"""

import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import rpa_oracle  # noqa: E402
from oracle.page_attention_oracle import page_attention_strict  # noqa: E402
from oracle.ragged_decode_oracle import ragged_decode_strict  # noqa: E402
from oracle.rpa_v3_oracle import rpa_v3  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))


def bf(x):
    return rpa_oracle.bf16_round(np.asarray(x, dtype=np.float32))


def rpa_case(seed, q_lens, kv_lens, Hq, Hkv, D, page, pps, window=None, cap=None):
    rng = np.random.default_rng(seed)
    S = len(q_lens)
    P = S * pps + 1
    T = int(sum(q_lens)) + 8
    q = bf(rng.standard_normal((T, Hq, D)))
    kv = bf(rng.standard_normal((P, page, 2 * Hkv, D)))
    bt = rng.permutation(P)[: S * pps].reshape(S, pps).astype(np.int32)
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    ctx = np.asarray(kv_lens, np.int32)
    ns = np.array([S], np.int32)
    scale = float(D) ** -0.5
    out = rpa_oracle.rpa_strict(q, kv, ctx, bt, qsl, ns, softmax_scale=scale, sliding_window=window, logits_soft_cap=cap)
    return dict(queries=rpa_oracle.bf16_bits(q), kv_pages=rpa_oracle.bf16_bits(kv), context_lens=ctx, block_tables=bt,
                query_start_loc=qsl, num_seqs=ns, softmax_scale=np.float32(scale),
                sliding_window=np.int32(window or 0), logits_soft_cap=np.float32(cap or 0.0),
                expected=rpa_oracle.bf16_bits(out))


def main():
    np.savez_compressed(os.path.join(HERE, "rpa_mixed.npz"),
                        **rpa_case(1, [1, 40, 3, 0, 1], [70, 100, 33, 5, 16], 4, 1, 128, 16, 7))
    np.savez_compressed(os.path.join(HERE, "rpa_window_cap_d256.npz"),
                        **rpa_case(2, [1, 1, 24], [120, 17, 60], 2, 1, 256, 16, 8, window=48, cap=30.0))

    rng = np.random.default_rng(3)
    q_lens, kv_lens, Hq, Hkv, D, page, pps = [2, 1, 20], [30, 64, 20], 4, 1, 128, 16, 4
    S, P, T = 3, 3 * 4 + 1, 23 + 8
    q, k, v = (bf(rng.standard_normal((T, h, D))) for h in (Hq, Hkv, Hkv))
    cache = bf(rng.standard_normal((P, page, Hkv, 2, D)))
    bt = rng.permutation(P)[: S * pps].astype(np.int32)
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    lens = np.asarray(kv_lens, np.int32)
    dist = np.array([0, 0, S], np.int32)
    out, new = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, softmax_scale=D ** -0.5)
    np.savez_compressed(os.path.join(HERE, "rpa_v3.npz"), queries=rpa_oracle.bf16_bits(q), keys=rpa_oracle.bf16_bits(k),
                        values=rpa_oracle.bf16_bits(v), kv_cache=rpa_oracle.bf16_bits(cache), kv_lens=lens,
                        block_tables=bt, query_start_loc=qsl, distribution=dist, softmax_scale=np.float32(D ** -0.5),
                        expected=rpa_oracle.bf16_bits(out), expected_cache=rpa_oracle.bf16_bits(new))

    # the same operation with a float8_e4m3fn cache (values stored as float16, which holds every e4m3 value exactly)
    rng = np.random.default_rng(13)
    f8 = rpa_oracle.fp8_e4m3fn_round
    q_lens, kv_lens, Hq, Hkv, D, page, pps = [3, 1, 24], [40, 64, 24], 4, 2, 128, 16, 4
    S, P, T = 3, 3 * 4 + 1, 28 + 4
    q = bf(rng.standard_normal((T, Hq, D)))
    k, v = (f8(rng.standard_normal((T, Hkv, D))) for _ in range(2))
    cache = f8(rng.standard_normal((P, page, 2 * Hkv // 4, 4, D)))
    bt = rng.permutation(P)[: S * pps].astype(np.int32)
    qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
    lens = np.asarray(kv_lens, np.int32)
    dist = np.array([0, 0, S], np.int32)
    kw = dict(softmax_scale=D ** -0.5, q_scale=0.05, k_scale=0.5, v_scale=2.0)
    out, new = rpa_v3(q, k, v, cache, lens, bt, qsl, dist, cache_dtype="float8_e4m3fn", query_dtype="bfloat16", **kw)
    assert all(np.array_equal(a.astype(np.float16).astype(np.float32), a) for a in (k, v, cache, new))
    np.savez_compressed(os.path.join(HERE, "rpa_v3_e4m3.npz"), queries=rpa_oracle.bf16_bits(q), keys=k.astype(np.float16),
                        values=v.astype(np.float16), kv_cache=cache.astype(np.float16), kv_lens=lens, block_tables=bt,
                        query_start_loc=qsl, distribution=dist, expected=rpa_oracle.bf16_bits(out),
                        expected_cache=new.astype(np.float16), **{n: np.float32(x) for n, x in kw.items()})

    rng = np.random.default_rng(4)
    ctx = np.array([1, 17, 100, 64], np.int32)
    nb, bs, mb = 4 * 7, 16, 7
    q = bf(rng.standard_normal((4, 4, 128)))
    kc, vc = (bf(rng.standard_normal((nb, 1, bs, 128))) for _ in range(2))
    bt = rng.permutation(nb).reshape(4, mb).astype(np.int32)
    out = page_attention_strict(q, kc, vc, ctx, bt, attn_scale=128 ** -0.5)
    np.savez_compressed(os.path.join(HERE, "page_attention.npz"), query=rpa_oracle.bf16_bits(q),
                        key_cache=rpa_oracle.bf16_bits(kc), value_cache=rpa_oracle.bf16_bits(vc), context_lens=ctx,
                        block_tables=bt, attn_scale=np.float32(128 ** -0.5), expected=rpa_oracle.bf16_bits(out))

    rng = np.random.default_rng(5)
    q = bf(rng.standard_normal((4, 4, 128)))
    k, v = (bf(rng.standard_normal((4, 96, 1, 128))) for _ in range(2))
    start, end = np.array([0, 3, 0, 40], np.int32), np.array([96, 50, 1, 41], np.int32)
    out = ragged_decode_strict(q, k, v, start, end, softmax_scale=128 ** -0.5, block_size=128)
    np.savez_compressed(os.path.join(HERE, "ragged_decode.npz"), query=rpa_oracle.bf16_bits(q), key=rpa_oracle.bf16_bits(k),
                        value=rpa_oracle.bf16_bits(v), sequence_start=start, sequence_end=end,
                        softmax_scale=np.float32(128 ** -0.5), block_size=np.int32(128),
                        expected=rpa_oracle.bf16_bits(out))

    # attention sinks: three biased positions, a window that leaves the sink range outside, starts inside and past
    # the biased positions, an empty sequence
    rng = np.random.default_rng(6)
    q = bf(rng.standard_normal((4, 4, 128)))
    k, v = (bf(rng.standard_normal((4, 96, 2, 128))) for _ in range(2))
    start, end = np.array([0, 1, 40, 90], np.int32), np.array([96, 50, 40, 96], np.int32)
    aux = np.array([[1.5, -0.75, 0.5], [0.0, 2.0, -1.0]], np.float32)
    out = ragged_decode_strict(q, k, v, start, end, softmax_scale=128 ** -0.5, block_size=128, sliding_window=(9, 0),
                               softmax_aux=aux)
    np.savez_compressed(os.path.join(HERE, "ragged_decode_sinks.npz"), query=rpa_oracle.bf16_bits(q),
                        key=rpa_oracle.bf16_bits(k), value=rpa_oracle.bf16_bits(v), sequence_start=start,
                        sequence_end=end, softmax_scale=np.float32(128 ** -0.5), block_size=np.int32(128),
                        window_left=np.int32(9), softmax_aux=aux, expected=rpa_oracle.bf16_bits(out))


if __name__ == "__main__":
    main()
