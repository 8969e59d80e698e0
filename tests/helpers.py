"""Shared test plumbing: tensor <-> numpy conversion and oracle invocation."""

import numpy as np
import torch

from ejkernel_amd.workloads import make_batch
from oracle import rpa_oracle

BF16_MAX_ABS = 2e-2   # tolerance of the bf16 path against the strict restatement
BF16_MEAN_ABS = 2e-3
F32_MAX_ABS = 1e-5    # tolerance of the fp32 path against the float64 evaluation


def to_np(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.dtype in (torch.bfloat16, torch.float8_e4m3fn, torch.float8_e5m2):
        return t.to(torch.float32).numpy()
    return t.numpy()


def host_view(batch):
    """The batch as the oracle should see it: on the CPU, and with only the referenced pages when the pool is large."""
    from ejkernel_amd.workloads import compact_for_host

    S = int(batch.num_seqs.reshape(-1)[0])
    page = batch.kv_pages.shape[1]
    used = int(sum(-(-int(k) // page) for k in batch.kv_lens[:S]))
    if batch.kv_pages.shape[0] > 2 * used + 64:
        return compact_for_host(batch, range(S))
    return batch


def oracle_args(batch):
    batch = host_view(batch)
    return (to_np(batch.queries), to_np(batch.kv_pages), to_np(batch.context_lens), to_np(batch.block_tables),
            to_np(batch.query_start_loc), to_np(batch.num_seqs))


def io_dtype(batch):
    return "bfloat16" if batch.queries.dtype == torch.bfloat16 else "float32"


def run_strict(batch, compute_dtype=None, softmax_aux=None, aux_dtype="float32"):
    """`aux_dtype`: the dtype the reference would hold `softmax_aux` in (float32 is what the device ABI takes; sinks
    as narrow as a bf16 carry keep the reference's whole epilogue in bf16)."""
    dt = io_dtype(batch)
    return rpa_oracle.rpa_strict(*oracle_args(batch), softmax_scale=batch.softmax_scale,
                                 logits_soft_cap=batch.logits_soft_cap, compute_dtype=compute_dtype or dt,
                                 sliding_window=batch.sliding_window, softmax_aux=softmax_aux, io_dtype=dt,
                                 aux_dtype=aux_dtype)


def run_exact(batch, softmax_aux=None):
    return rpa_oracle.rpa_exact(*oracle_args(batch), softmax_scale=batch.softmax_scale,
                                logits_soft_cap=batch.logits_soft_cap, sliding_window=batch.sliding_window,
                                softmax_aux=softmax_aux)


def err_stats(a, b, rows):
    d = np.abs(np.asarray(a, np.float64)[:rows] - np.asarray(b, np.float64)[:rows])
    return float(d.max(initial=0.0)), float(d.mean()) if d.size else 0.0


def assert_bf16_parity(out, ref, rows, what=""):
    mx, mean = err_stats(out, ref, rows)
    assert np.isfinite(np.asarray(out)[:rows]).all(), f"{what}: non-finite output"
    assert mx <= BF16_MAX_ABS and mean <= BF16_MEAN_ABS, f"{what}: max-abs {mx:.4g} mean-abs {mean:.4g}"
    return mx, mean


def assert_bf16_parity_stepwise(out, ref, what="", exact=None):
    """The parity bound, widened to two bf16 steps of the value where that is larger: rows that see one or two keys
    return values of magnitude 2..8, whose step is 0.016..0.031, and the reference's chain of bf16 roundings puts its
    restatement up to 1.5 steps from the float64 value there.  Every path rounds where the reference does and is held to
    this bound as it stands.

    `exact` (the float64 evaluation) is given only for a reference program that normalises the probabilities before
    the product with V (`ragged_decode_attention`: e / l, the product, l times it and the division are four bf16
    roundings after the exponential, where a one-pass kernel divides once in fp32): there an element may sit three steps
    from the restatement if it is at least as close to the float64 value as the restatement is."""
    ref = np.asarray(ref, np.float64)
    out64 = np.asarray(out, np.float64)
    d = np.abs(out64 - ref)
    step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref), 1e-30))) - 7)
    assert np.isfinite(np.asarray(out)).all(), f"{what}: non-finite output"
    over = d > np.maximum(BF16_MAX_ABS, 2 * step)
    if exact is not None and over.any():
        ex = np.asarray(exact, np.float64)
        over &= ~((d <= np.maximum(BF16_MAX_ABS, 3 * step) + 1e-12) & (np.abs(out64 - ex) <= np.abs(ref - ex)))
    assert not over.any() and d.mean() <= BF16_MEAN_ABS, f"{what}: max-abs {d.max():.4g} mean-abs {d.mean():.4g}"


def random_rpa_batch(seed, device, head_dims=(64, 128, 256)):
    """A seeded draw over the argument space: head counts, head_dim, page size, ragged lengths, window, cap."""
    rng = np.random.default_rng(seed)
    hq, hkv = [(8, 2), (4, 4), (16, 2), (32, 8), (8, 1), (12, 4)][rng.integers(6)]
    D = int(rng.choice(list(head_dims)))
    page = int(rng.choice([4, 8, 16, 32, 64]))
    n = int(rng.integers(1, 9))
    kinds = rng.integers(0, 5, size=n)
    q_lens, kv_lens = [], []
    for k in kinds:
        if k == 0:                       # absent query: the sequence contributes nothing
            q, prior = 0, int(rng.integers(0, 40))
        elif k == 1:                     # decode
            q, prior = 1, int(rng.integers(0, 400))
        elif k == 2:                     # a few rows
            q, prior = int(rng.integers(2, 9)), int(rng.integers(0, 200))
        elif k == 3:                     # prefill chunk with earlier context
            q, prior = int(rng.integers(20, 150)), int(rng.integers(0, 300))
        else:                            # prefill from scratch
            q, prior = int(rng.integers(20, 150)), 0
        q_lens.append(q)
        kv_lens.append(q + prior)
    pps = -(-max(max(kv_lens), 1) // page) + int(rng.integers(0, 3))
    if pps >= 64:  # the reference's block-table windows of 64 entries clamp at the end of a row that is not a multiple
        pps = -(-pps // 64) * 64  # of 64 long and then read the wrong pages: the restatement reproduces that, avoid it
    window = None if rng.random() < 0.5 else int(rng.integers(1, 200))
    cap = None if rng.random() < 0.6 else float(rng.choice([5.0, 20.0, 50.0]))
    extra = int(rng.integers(0, 4))
    b = make_batch(q_lens, kv_lens, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, page_size=page, pages_per_seq=pps,
                   seed=seed, device=device, sliding_window=window, logits_soft_cap=cap, max_num_seqs=n + extra)
    return b, f"seed {seed}: {hq}/{hkv} D={D} page={page} q={q_lens} kv={kv_lens} W={window} cap={cap}"


def random_serving_batch(seed, device):
    """A seeded draw over the shapes of a serving step: one to three long chunks after contexts of up to 8000 tokens
    with up to 70 decode steps beside them, small batches of decode steps, or a few decode sequences of up to 70000 keys;
    sometimes inside padded static shapes, sometimes with the tile shape named.  Returns the batch, the sinks (or
    None), the config hint (or 0) and a description."""
    rng = np.random.default_rng(seed)
    regime = ["chunks", "chunks", "small_decode", "long_decode"][rng.integers(4)]
    hq, hkv = [(32, 8), (16, 4), (8, 2), (16, 2), (8, 8)][rng.integers(5)]
    D = int(rng.choice([128, 128, 128, 64, 256]))
    page = int(rng.choice([16, 32, 64]))
    window = None if rng.random() < 0.7 else int(rng.integers(16, 3000))
    cap = None if rng.random() < 0.8 else 30.0
    aux = None if rng.random() < 0.8 else rng.standard_normal((hq, 1)).astype(np.float32)
    if regime == "chunks":
        n_ch = int(rng.integers(1, 4))
        q = [int(rng.integers(60, 1100 // n_ch + 60)) for _ in range(n_ch)]
        kv = [qq + int(rng.choice([0, rng.integers(0, 600), rng.integers(0, 8000)])) for qq in q]
        n_dec = int(rng.choice([0, 0, rng.integers(1, 8), rng.integers(8, 72)]))
        q += [1] * n_dec
        kv += [int(rng.integers(1, 4000)) for _ in range(n_dec)]
    elif regime == "small_decode":
        n = int(rng.integers(1, 72))
        q = [int(rng.choice([1, 1, 1, rng.integers(1, 5)])) for _ in range(n)]
        kv = [max(qq, int(rng.integers(1, rng.choice([64, 600, 3000])))) for qq in q]
    else:
        q = [1] * int(rng.integers(1, 5))
        kv = [int(rng.integers(1, rng.choice([9000, 70000]))) for _ in q]
    order = rng.permutation(len(q))
    q, kv = [q[i] for i in order], [kv[i] for i in order]
    pps = -(-max(kv) // page)
    pps = pps if pps < 64 else -(-pps // 64) * 64
    kw = {}
    if rng.random() < 0.4:   # a caller's padded static shapes
        kw = dict(max_num_seqs=int(rng.choice([len(q) + 3, 256, 512])), pool_seqs=len(q),
                  total_tokens=int(max(((sum(q) + 7) // 8) * 8 + 8, rng.choice([2048, 8192]))))
    hint = int(rng.choice([0, 0, 128, 256])) if regime == "chunks" else 0
    b = make_batch(q, kv, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, page_size=page, pages_per_seq=pps, seed=seed,
                   device=device, sliding_window=window, logits_soft_cap=cap, **kw)
    what = (f"seed {seed} {regime}: {hq}/{hkv} D={D} page={page} q={q} kv={kv} W={window} cap={cap} "
            f"sinks={aux is not None} pad={kw} hint={hint}")
    return b, aux, hint, what


def two_key_cap_batch(device="cpu", head_dim=16, dtype=torch.bfloat16):
    """One query row over two keys with the soft cap 23.7, which bf16 does not hold (the weakly typed scalar becomes
    23.75 before it divides and multiplies, _xla_impl_fwd.py:125-126).  q . k is 20 for key 0 and 16 for key 1
    (scale 1), V is 0 and 8.  By hand, every op rounded to bf16: 20 / 23.75 -> 0.84375, tanh -> 0.6875, * 23.75 ->
    16.375; 16 / 23.75 -> 0.671875, tanh -> 0.5859375, * 23.75 -> 13.9375; p1 = bf16(exp(-2.4375)) = 0.08740234375,
    l = bf16(1.08740234375) = 1.0859375, o = 8 p1 = 0.69921875, out = bf16(o / l) = 0.64453125.  With the cap left at
    23.7 the two logits become 16.25 and 13.875 and the output 0.6796875; a device that normalises with the fp32 row sum
    (1.08740234375) lands on 0.64453125 as well."""
    b = make_batch([1], [2], num_q_heads=1, num_kv_heads=1, head_dim=head_dim, page_size=4, pages_per_seq=1, seed=0,
                   dtype=dtype, device=device, logits_soft_cap=23.7, softmax_scale=1.0)
    pg = int(b.block_tables[0, 0])
    b.queries.zero_()
    b.queries[0, 0, 0] = 4.0
    b.kv_pages[pg].zero_()
    b.kv_pages[pg, 0, 0, 0] = 5.0   # K of key 0
    b.kv_pages[pg, 1, 0, 0] = 4.0   # K of key 1
    b.kv_pages[pg, 1, 1, :] = 8.0   # V of key 1 (V of key 0 is zero)
    return b, 0.64453125
