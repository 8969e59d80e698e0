"""Shared test plumbing: tensor <-> numpy conversion and oracle invocation."""

import numpy as np
import torch

from oracle import rpa_oracle

BF16_MAX_ABS = 2e-2   # tolerance of the bf16 path against the strict restatement
BF16_MEAN_ABS = 2e-3
F32_MAX_ABS = 1e-5    # tolerance of the fp32 path against the float64 evaluation


def to_np(t: torch.Tensor) -> np.ndarray:
    t = t.detach().cpu()
    if t.dtype == torch.bfloat16:
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


def run_strict(batch, compute_dtype=None, softmax_aux=None):
    dt = io_dtype(batch)
    return rpa_oracle.rpa_strict(*oracle_args(batch), softmax_scale=batch.softmax_scale,
                                 logits_soft_cap=batch.logits_soft_cap, compute_dtype=compute_dtype or dt,
                                 sliding_window=batch.sliding_window, softmax_aux=softmax_aux, io_dtype=dt)


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
