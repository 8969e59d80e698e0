"""Benchmark of the ragged paged attention forward on one MI355X.

``python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]`` runs W untimed and K
timed forward passes of one synthetic batch (already resident in HBM) and prints ONE JSON line.
A "step" is one pass of the op over the whole ragged batch.  The default workload is the
Llama-3-8B-shape decode batch (256 sequences x 1 token, kv 512..8192, 32 q / 8 kv heads,
head_dim 128, page 16, 160k-page pool); the metric is query tokens per second, with the achieved
fraction of the HBM roofline of the attention kernel and, beside it, the CPU restatement of the
reference's XLA path timed on this host on a bounded sample of the same batch.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


# HBM bytes per launch as the FETCH_SIZE / WRITE_SIZE counter passes measured them (each counter scaled by what it reads
# for a plain device copy of known size): profiles/hbm_traffic.json, written by `python -m ejkernel_amd.hbm_traffic`
# from the counter files of a profile run.  A workload without an entry reports null.
def measured_traffic_bytes(workload: str):
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            entry = json.load(f).get(workload)
        return None if entry is None else float(entry["bytes"])
    except (OSError, ValueError, KeyError):
        return None


# The configurations of the benchmark besides the headline one, measured in the same run (entries of "configs").  The
# two other bandwidth-bound streams come first: how fast a stream runs depends by a few per cent on the memory its pool
# gets, and pools allocated early in a process get what a process of their own would (gemma2_local 0.386 ms as the
# second workload of a process, 0.392-0.398 ms as the fifth; 0.380 ms alone).
EXTRA_CONFIGS = ["gemma2_local", "decode_long_context", "decode_small", "mixed_prefill_decode", "mixed_prefill_only",
                 "prefill_single_16k",
                 # one request's chunked prefill, alone and beside 64 decode steps: latency, like decode_small
                 "prefill_chunk_after_8k", "chunk_beside_decodes",
                 # What a serving caller with padded static shapes gets (max_num_seqs 512, query rows rounded up to
                 # 8192 / 16384, num_seqs as is): the library's own choice of kernel instantiation, made from those
                 # shapes, and the choice the caller names through RaggedPageAttentionConfig.num_queries_per_block.
                 ("decode_llama3_8b_padded", None), ("decode_llama3_8b_padded", 16),
                 ("mixed_prefill_decode_padded", None), ("mixed_prefill_decode_padded", 128),
                 ("mixed_prefill_only_padded", None), ("mixed_prefill_only_padded", 256)]
# Prompts too long for the CPU restatement: checked on a prefix against it and on sampled rows against float64
# (long_prompt_parity).  prefill_single_16k is not one of the five benchmark configurations: it shows the prefill tile
# where a tile walks up to 16384 keys and what a tile costs besides its key loop no longer counts.
LONG_PROMPT_CONFIGS = ("prefill_single_16k", "prefill_long")


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="decode_llama3_8b")
    ap.add_argument("--op", default="rpa", choices=["rpa", "rpa_v3", "page_attention", "ragged_decode"],
                    help="rpa = ragged_page_attention (the headline path); rpa_v3 = ragged_page_attention_v3 on the same "
                         "workload: every query token also brings a new K/V row that is written into the cache first; "
                         "page_attention = the decode workloads (decode_small, decode_llama3_8b) with separate K and V "
                         "caches of [blocks, kv heads, block, head_dim]; ragged_decode = ragged_decode_attention on the "
                         "same lengths with contiguous K and V of [batch, seq_len, kv heads, head_dim]")
    ap.add_argument("--cache-dtype", default="same", choices=["same", "fp8"],
                    help="--op rpa_v3: dtype of the cache and of the new K/V rows; fp8 = float8_e4m3fn with bf16 queries")
    ap.add_argument("--sinks", type=int, default=0,
                    help="--op ragged_decode: attention sinks (softmax_aux of this many biases, shared by all heads)")
    ap.add_argument("--window", type=int, default=0,
                    help="--op ragged_decode: sliding_window=(WINDOW - 1, 0), i.e. the last WINDOW keys (0 = none)")
    ap.add_argument("--scale", type=float, default=1.0, help="shrink the workload (debugging only)")
    ap.add_argument("--cpu-seqs", type=int, default=0, help="sequences in the CPU sample (0 = pick for ~10-30 s)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="only the headline workload: skip the other benchmark configurations (the \"configs\" array)")
    ap.add_argument("--copy-probe", type=int, default=0, metavar="MIB",
                    help="instead of the benchmark, run a plain device copy of MIB MiB --steps times (a kernel of "
                         "known traffic, used to scale the FETCH_SIZE / WRITE_SIZE counters)")
    ap.add_argument("--sustain", type=float, default=0.0, metavar="SECONDS",
                    help="instead of the benchmark, launch the workload (or the --gemm-probe product) back to back for "
                         "SECONDS and print the time per launch with the board's power sensor and power cap (hwmon)")
    ap.add_argument("--gemm-probe", type=int, default=0, metavar="N",
                    help="instead of the benchmark, time the vendor library's bf16 N x N x N matrix product (what the "
                         "matrix cores of this box sustain under its power limit; context for the MFMA-bound figures)")
    return ap.parse_args()


def cpu_sample_and_parity(batch, out, want_baseline, want_parity, n_seqs, budget_s=12.0):
    """Times the CPU restatement of the reference's XLA path (oracle/rpa_oracle.c, OpenMP over all host cores)
    on a bounded sample of the batch's sequences and checks the device rows of that sample against it."""
    import numpy as np

    from ejkernel_amd.workloads import compact_for_host
    from oracle import rpa_oracle_c
    from tests.helpers import err_stats, oracle_args, run_exact, to_np

    S = len(batch.q_lens)
    rng = np.random.default_rng(0)
    cand = [int(s) for s in rng.permutation(S) if batch.q_lens[s] > 0]
    if batch.sliding_window:
        # the reference program turns rows NaN where a 64-page KV block lies left of the window (those are compared with
        # the float64 evaluation): the sequences short enough to have no such block go first, every second place
        limit = batch.sliding_window + 64 * batch.meta["page_size"]
        short = [s for s in cand if batch.kv_lens[s] < limit]
        rest = [s for s in cand if batch.kv_lens[s] >= limit]
        cand = [x for pair in zip(short, rest) for x in pair] + short[len(rest):] + rest[len(short):]
    threads = rpa_oracle_c.max_threads()

    def run(ids):
        sub = compact_for_host(batch, sorted(ids))
        args = oracle_args(sub)
        t0 = time.perf_counter()
        ref = rpa_oracle_c.rpa_strict_c(*args, softmax_scale=sub.softmax_scale, logits_soft_cap=sub.logits_soft_cap,
                                        sliding_window=sub.sliding_window, io_dtype="bfloat16", threads=threads)
        return sub, ref, time.perf_counter() - t0

    if n_seqs <= 0:
        # probe with a few sequences, then size the sample for about `budget_s` seconds of CPU work
        probe = cand[:max(1, min(len(cand), threads // 8 or 1))]
        sub, _, dt = run(probe)
        work = lambda ids: float(sum((-(-int(batch.q_lens[s]) // 8)) * int(batch.kv_lens[s]) for s in ids))  # noqa: E731
        rate = work(probe) / max(dt, 1e-3)
        n_seqs, acc = 0, 0.0
        for s in cand:
            acc += work([s])
            n_seqs += 1
            if acc / rate > budget_s:
                break
    ids = cand[:max(1, n_seqs)]
    sub, ref, dt = run(ids)
    reps = 1
    while dt * reps < budget_s and reps < 20:  # a fast host: repeat the sample until ~budget_s of CPU work is timed
        _, _, dt_k = run(ids)
        dt = (dt * reps + dt_k) / (reps + 1)
        reps += 1
    rows = sub.total_valid_tokens
    res = {}
    if want_parity:
        got = to_np(out[sub.meta["rows"].to(out.device)])
        bad = np.isnan(ref[:rows]).any(axis=(1, 2))
        if bad.any():  # NaN rows of the reference program (window defect): compare with the float64 evaluation
            # only the sequences that have such rows are evaluated (dense float64 is slow on long chunks), and a line on
            # stderr says so: minutes of silent host work look like a hang from outside
            ref = ref.copy()
            starts = np.concatenate([[0], np.cumsum(sub.q_lens)])
            order = sorted(ids)
            for k in range(len(order)):
                r0, r1 = int(starts[k]), int(starts[k + 1])
                if not bad[r0:r1].any():
                    continue
                print(f"bench.py: float64 evaluation of sequence {order[k]} ({r1 - r0} rows the reference program turns NaN in part)",
                      file=sys.stderr, flush=True)
                one = compact_for_host(batch, [order[k]])
                ex = run_exact(one)[: r1 - r0]
                seg = ref[r0:r1]
                seg[bad[r0:r1]] = ex[bad[r0:r1]]
        mx, mean = err_stats(got, ref, rows)
        over = int((np.abs(np.asarray(got[:rows], np.float64) - np.asarray(ref[:rows], np.float64)) > 2e-2).sum())
        res["parity"] = {"max_abs": mx, "mean_abs": mean, "rows": rows, "oracle_nan_rows": int(bad.sum()),
                         "elements_over_2e-2": over, "ok": bool(mx <= 2e-2 and mean <= 2e-3)}
    if want_baseline:
        res["cpu_baseline"] = {
            "value": rows / dt, "unit": "tokens/s", "cores": int(threads), "kind": "port",
            "sample": f"{len(ids)} of {S} sequences ({rows} query tokens, {int(sub.kv_lens.sum())} kv tokens), mean of "
                      f"{reps} runs of {dt:.2f} s; C restatement of the reference's XLA path (8-row query blocks, 64-page KV blocks, "
                      f"bf16 rounding points), OpenMP over {threads} threads",
        }
    return res


def long_prompt_parity(batch, out, prefix_tokens=768, sampled_tokens=48):
    """Parity for a workload of few, very long prompts, which the CPU restatement cannot walk in seconds.  Causal
    attention makes the first `prefix_tokens` rows of a prompt the attention of that prefix alone: those rows are checked
    against the restatement of the reference program on the prefix as a prompt of its own (the parity bound, widened to
    two bf16 steps of the value where that is larger; the record also carries the count against the plain 2e-2 with
    the smallest and largest |reference value| among those elements and the most keys any of their rows sees).  Rows deep
    in the prompt are checked, `sampled_tokens` positions per prompt, against a float64 evaluation on the device (plain
    torch: gather the prompt's K / V rows, scores, softmax, product) with the bound the tests use against float64."""
    import numpy as np
    import torch

    from ejkernel_amd.workloads import Batch
    from oracle import rpa_oracle_c
    from tests.helpers import err_stats, oracle_args, to_np

    m = batch.meta
    G = m["num_q_heads"] // m["num_kv_heads"]
    page = m["page_size"]
    cu = batch.query_start_loc.cpu().numpy()
    worst = {"prefix_max_abs": 0.0, "prefix_mean_abs": 0.0, "deep_max_abs": 0.0, "deep_mean_abs": 0.0}
    rows_prefix = rows_deep = over_bound = over_plain = 0
    plain_min_value, plain_max_value, plain_max_keys = None, None, 0
    rng = np.random.default_rng(0)
    for s in range(len(batch.q_lens)):
        L, q0 = int(batch.kv_lens[s]), int(cu[s])
        if int(batch.q_lens[s]) != L:
            raise ValueError("long_prompt_parity takes prompts from scratch")
        n0 = min(prefix_tokens, L)
        n_pg = -(-n0 // page)
        phys = batch.block_tables[s, :n_pg].long()
        t_alloc = ((n0 + 7) // 8) * 8 + 8
        q = torch.zeros((t_alloc,) + tuple(batch.queries.shape[1:]), dtype=batch.queries.dtype)
        q[:n0] = batch.queries[q0:q0 + n0].cpu()
        sub = Batch(queries=q, kv_pages=batch.kv_pages[phys].cpu(), context_lens=torch.tensor([n0], dtype=torch.int32),
                    block_tables=torch.arange(n_pg, dtype=torch.int32)[None], query_start_loc=torch.tensor([0, n0], dtype=torch.int32),
                    num_seqs=torch.tensor([1], dtype=torch.int32), softmax_scale=batch.softmax_scale,
                    sliding_window=batch.sliding_window, logits_soft_cap=batch.logits_soft_cap, q_lens=np.array([n0]),
                    kv_lens=np.array([n0]), name=batch.name + "/prefix", meta=dict(m))
        ref = rpa_oracle_c.rpa_strict_c(*oracle_args(sub), softmax_scale=sub.softmax_scale, logits_soft_cap=sub.logits_soft_cap,
                                        sliding_window=sub.sliding_window, io_dtype="bfloat16", threads=rpa_oracle_c.max_threads())
        got = to_np(out[q0:q0 + n0])
        mx, mean = err_stats(got, ref, n0)
        worst["prefix_max_abs"], worst["prefix_mean_abs"] = max(worst["prefix_max_abs"], mx), max(worst["prefix_mean_abs"], mean)
        # The first rows of a prompt see one or two keys and return values of magnitude 2..8, whose bf16 step is
        # 0.016..0.031: the bound is the parity bound or two bf16 steps of the value, whichever is larger (the bound of
        # tests.helpers.assert_bf16_parity_stepwise, which the prefill tiles are held to in the tests).
        ref64 = np.asarray(ref[:n0], np.float64)
        step = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(ref64), 1e-30))) - 7)
        diff = np.abs(np.asarray(got[:n0], np.float64) - ref64)
        over_bound += int((diff > np.maximum(2e-2, 2 * step)).sum())
        # the same count against the plain bound, with what the elements over it have in common: the magnitude of the
        # reference value there (a bf16 step of 2e-2 / 1.28 or more needs |value| >= 2) and how many keys the row sees
        plain = diff > 2e-2
        if plain.any():
            over_plain += int(plain.sum())
            vals = np.abs(ref64[plain])
            plain_min_value = float(vals.min()) if plain_min_value is None else min(plain_min_value, float(vals.min()))
            plain_max_value = float(vals.max()) if plain_max_value is None else max(plain_max_value, float(vals.max()))
            first_key = 0 if not batch.sliding_window else np.maximum(0, np.nonzero(plain)[0] + 1 - batch.sliding_window)
            plain_max_keys = max(plain_max_keys, int((np.nonzero(plain)[0] + 1 - first_key).max()))
        rows_prefix += n0
        # rows deep in the prompt, in float64 on the device
        pages = batch.kv_pages[batch.block_tables[s, : -(-L // page)].long()]          # [pages, page, 2 Hkv, D]
        kv = pages.reshape(-1, 2 * m["num_kv_heads"], m["head_dim"])[:L].double()
        k, v = kv[:, 0::2], kv[:, 1::2]                                                 # [L, Hkv, D]
        pos = np.unique(np.concatenate([rng.integers(n0, L, size=sampled_tokens - 1), [L - 1]])) if L > n0 else np.array([L - 1])
        for t in pos:
            qt = batch.queries[q0 + int(t)].double().reshape(m["num_kv_heads"], G, m["head_dim"])
            sc = torch.einsum("hgd,khd->hgk", qt, k[: int(t) + 1]) * batch.softmax_scale
            if batch.logits_soft_cap:
                sc = batch.logits_soft_cap * torch.tanh(sc / batch.logits_soft_cap)
            if batch.sliding_window:
                sc[..., : max(0, int(t) + 1 - batch.sliding_window)] = -float("inf")
            ref_t = torch.einsum("hgk,khd->hgd", torch.softmax(sc, dim=-1), v[: int(t) + 1]).reshape(m["num_q_heads"], m["head_dim"])
            d = (out[q0 + int(t)].double() - ref_t).abs()
            worst["deep_max_abs"] = max(worst["deep_max_abs"], float(d.max()))
            worst["deep_mean_abs"] += float(d.mean())
            rows_deep += 1
        del pages, kv, k, v
    worst["deep_mean_abs"] /= max(rows_deep, 1)
    worst.update({"rows_prefix": rows_prefix, "rows_deep": rows_deep, "prefix_elements_over_bound": over_bound,
                  "prefix_elements_over_2e-2": over_plain, "over_2e-2_min_abs_value": plain_min_value,
                  "over_2e-2_max_abs_value": plain_max_value, "over_2e-2_max_visible_keys": plain_max_keys,
                  "ok": bool(over_bound == 0 and worst["prefix_mean_abs"] <= 2e-3 and
                             worst["deep_max_abs"] <= 4e-2 and worst["deep_mean_abs"] <= 2e-3)})
    return worst


def cpu_sample_and_parity_v3(batch, v3, out, want_baseline, want_parity, n_seqs, budget_s=12.0):
    """The same for ragged_page_attention_v3: the NumPy restatement of the reference program (oracle/rpa_v3_oracle.py)
    on a bounded sample of sequences, whose cache pages are taken as they were before the timed calls."""
    import numpy as np

    from ejkernel_amd.workloads import compact_for_host, to_v3
    from oracle.rpa_v3_oracle import rpa_v3
    from tests.helpers import err_stats, to_np

    try:
        from threadpoolctl import threadpool_info
        threads = max([int(i.get("num_threads", 1)) for i in threadpool_info()] or [1])
    except Exception:  # pragma: no cover
        threads = 1
    S = len(batch.q_lens)
    rng = np.random.default_rng(0)
    cand = [int(s) for s in rng.permutation(S) if batch.q_lens[s] > 0]

    def run(ids):
        sub = compact_for_host(batch, sorted(ids))
        fp8 = v3.kv_cache.dtype != v3.queries.dtype
        sv = to_v3(sub, cache_dtype=v3.kv_cache.dtype if fp8 else None)
        rows_idx = sub.meta["rows"]
        sv.keys[: len(rows_idx)] = v3.keys[rows_idx.to(v3.keys.device)].cpu()
        sv.values[: len(rows_idx)] = v3.values[rows_idx.to(v3.keys.device)].cpu()
        a = [to_np(x) for x in sv.args()]
        t0 = time.perf_counter()
        dt = dict(cache_dtype="float8_e4m3fn", query_dtype="bfloat16") if fp8 else {}
        ref, _ = rpa_v3(*a, **sv.kwargs(), **dt)
        return sub, ref, time.perf_counter() - t0

    if n_seqs <= 0:
        sub, _, dt = run(cand[:1])
        work = lambda ids: float(sum(int(batch.q_lens[s]) * int(batch.kv_lens[s]) + int(batch.kv_lens[s]) for s in ids))  # noqa: E731
        rate = work(cand[:1]) / max(dt, 1e-3)
        n_seqs, acc = 0, 0.0
        for s in cand:
            acc += work([s])
            n_seqs += 1
            if acc / rate > budget_s:
                break
    ids = cand[:max(1, n_seqs)]
    sub, ref, dt = run(ids)
    rows = sub.total_valid_tokens
    res = {}
    if want_parity:
        got = to_np(out[sub.meta["rows"].to(out.device)])
        mx, mean = err_stats(got, ref, rows)
        res["parity"] = {"max_abs": mx, "mean_abs": mean, "rows": rows, "ok": bool(mx <= 2e-2 and mean <= 2e-3)}
    if want_baseline:
        res["cpu_baseline"] = {
            "value": rows / dt, "unit": "tokens/s", "cores": int(threads), "kind": "port",
            "sample": f"{len(ids)} of {S} sequences ({rows} query tokens, {int(sub.kv_lens.sum())} kv tokens), one run of "
                      f"{dt:.2f} s; NumPy restatement of the reference's v3 program (cache update, float32 dense attention per "
                      f"sequence on the visible keys), BLAS threads {threads}",
        }
    return res


def page_attention_main(args):
    """bench.py --op page_attention: the same contract as the default path, for the page_attention operation."""
    import numpy as np
    import torch

    from ejkernel_amd.modules import page_attention, ragged_decode_attention
    from ejkernel_amd.roofline import HBM_PEAK_GBPS, algorithmic_counts
    from ejkernel_amd.workloads import (WORKLOADS, page_attention_subset, page_attention_workload,
                                        ragged_decode_workload)

    dev = "cuda:0"
    contiguous = args.op == "ragged_decode"
    if contiguous:
        b = ragged_decode_workload(args.workload, device=dev, scale=args.scale)
        b.kv_lens = b.ends - b.starts
    else:
        b = page_attention_workload(args.workload, device=dev, scale=args.scale)
    m = b.meta
    S = len(b.kv_lens)
    counts = algorithmic_counts(np.ones(S, np.int64), b.kv_lens, num_q_heads=m["num_q_heads"],
                                num_kv_heads=m["num_kv_heads"], head_dim=m["head_dim"], page_size=m.get("page_size", 16))

    aux = torch.linspace(-1.0, 2.0, args.sinks, device=dev) if contiguous and args.sinks > 0 else None
    window = (args.window - 1, 0) if contiguous and args.window > 0 else None
    if contiguous and (aux is not None or window is not None):
        # keys a sequence reads: its last WINDOW ones plus the sink range
        seen = np.minimum(b.kv_lens, args.window) if window is not None else b.kv_lens
        b.kv_lens = np.minimum(b.kv_lens, seen + args.sinks)
        counts = algorithmic_counts(np.ones(S, np.int64), b.kv_lens, num_q_heads=m["num_q_heads"],
                                    num_kv_heads=m["num_kv_heads"], head_dim=m["head_dim"], page_size=16)

    def step():
        if contiguous:
            return ragged_decode_attention(*b.args(), aux, softmax_scale=b.softmax_scale, sliding_window=window)
        return page_attention(*b.args(), attn_scale=b.attn_scale)

    settle(step)
    for _ in range(args.warmup):
        out = step()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        starts[i].record()
        out = step()
        ends[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ev_ms = sorted(s.elapsed_time(e) for s, e in zip(starts, ends))
    kernel_ms = sum(ev_ms) / len(ev_ms)
    ms_per_step = wall * 1e3 / args.steps
    gbps = counts["bytes"] / (kernel_ms * 1e-3) / 1e9
    line = {
        "metric": "ragged-decode-attn tokens/s" if contiguous else "page-attn tokens/s", "value": S / (ms_per_step * 1e-3), "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "settle_s": SETTLE_S, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "op": args.op, "description": WORKLOADS[args.workload], "scale": args.scale,
                   "query_tokens": S, "num_seqs": S, "kv_tokens": int(b.kv_lens.sum()),
                   **({"sinks": args.sinks, "window": args.window} if contiguous else {})},
        "roofline": {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS,
                     "traffic": None, "kernel_ms_avg": kernel_ms, "kernel_ms_min": ev_ms[0],
                     "kernel_ms_median": ev_ms[len(ev_ms) // 2], "algorithmic_bytes": counts["bytes"],
                     "algorithmic_flops": counts["flops"], "gbps": gbps},
    }
    if not (args.no_cpu_baseline and args.no_parity):
        from oracle.page_attention_oracle import page_attention_strict
        from tests.helpers import err_stats, to_np

        try:
            from threadpoolctl import threadpool_info
            threads = max([int(i.get("num_threads", 1)) for i in threadpool_info()] or [1])
        except Exception:  # pragma: no cover
            threads = 1
        rng = np.random.default_rng(0)
        cand = [int(s) for s in rng.permutation(S)]
        n = args.cpu_seqs or min(S, 48)
        if contiguous:
            # The reference program is attention only for sequences inside one KV block, so it is timed and used as the
            # checker with a block that covers the sequence (fwd_params.kv_blocksize >= seq_len).
            from oracle.ragged_decode_oracle import ragged_decode_strict

            ids = torch.tensor(sorted(cand[:n]))
            a = [to_np(t[ids.to(dev)]) for t in b.args()]
            t0 = time.perf_counter()
            ref = ragged_decode_strict(*a, softmax_scale=b.softmax_scale, block_size=int(m["seq_len"]),
                                       sliding_window=window, softmax_aux=None if aux is None else to_np(aux))
            dt = time.perf_counter() - t0
            rows_idx, kv_tokens = ids, int(b.kv_lens[ids.numpy()].sum())
            what = ("NumPy restatement of the reference's XLA scan with one KV block per sequence (bf16 op by op)")
        else:
            sub = page_attention_subset(b, sorted(cand[:n]))
            a = [to_np(t) for t in sub.args()]
            t0 = time.perf_counter()
            ref = page_attention_strict(*a, attn_scale=b.attn_scale)
            dt = time.perf_counter() - t0
            rows_idx, kv_tokens = sub.meta["rows"], int(sub.kv_lens.sum())
            what = ("NumPy restatement of the reference's XLA program (every block-table entry gathered, one dense bf16 "
                    "softmax per sequence)")
        if not args.no_parity:
            mx, mean = err_stats(to_np(out[rows_idx.to(dev)]), ref, n)
            line["parity"] = {"max_abs": mx, "mean_abs": mean, "rows": n, "ok": bool(mx <= 2e-2 and mean <= 2e-3)}
        if not args.no_cpu_baseline:
            line["cpu_baseline"] = {
                "value": n / dt, "unit": "tokens/s", "cores": int(threads), "kind": "port",
                "sample": f"{n} of {S} sequences ({kv_tokens} kv tokens), one run of {dt:.2f} s; {what}, BLAS threads "
                          f"{threads}",
            }
    print(json.dumps(line))


SETTLE_S = 0.25


def settle(fn, seconds=SETTLE_S):
    """Untimed launches of `fn` back to back for `seconds` before the warm-up.  After an idle spell the device takes
    tens of launches to reach the clocks it then holds: the first 25 launches of the 512-token prefill chunks average
    0.40 ms, every later one 0.335 ms (the bandwidth-bound workloads differ by 1 %).  What is timed is the state a
    serving loop runs in; the JSON line says how long this phase was ("settle_s")."""
    import torch

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(20):
            fn()
        torch.cuda.synchronize()


def time_steps(step, steps, warmup, settle_s=SETTLE_S):
    """`warmup` untimed calls, then `steps` calls bracketed by synchronisation: wall time per step, the per-call
    durations between HIP events on the stream the op launches on (torch's current one), and the last output."""
    import torch

    settle(step, settle_s)
    out = None
    for _ in range(warmup):
        out = step()
    torch.cuda.synchronize()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        starts[i].record()
        out = step()
        ends[i].record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall * 1e3 / steps, sorted(s.elapsed_time(e) for s, e in zip(starts, ends)), out


def roofline_of(counts, ev_ms):
    """The roofline object of a workload: the bound its algorithmic bytes and flops put it under at MI355X's peaks,
    priced with the average kernel duration."""
    from ejkernel_amd.roofline import HBM_PEAK_GBPS, MFMA_BF16_PEAK_TFLOPS

    kernel_ms = sum(ev_ms) / len(ev_ms)
    gbps = counts["bytes"] / (kernel_ms * 1e-3) / 1e9
    tflops = counts["flops"] / (kernel_ms * 1e-3) / 1e12
    if counts["bytes"] / (HBM_PEAK_GBPS * 1e9) >= counts["flops"] / (MFMA_BF16_PEAK_TFLOPS * 1e12):
        roof = {"bound": "hbm", "achieved": gbps, "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": gbps / HBM_PEAK_GBPS}
    else:
        roof = {"bound": "mfma", "achieved": tflops, "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": tflops / MFMA_BF16_PEAK_TFLOPS}
    roof.update({"traffic": None, "kernel_ms_avg": kernel_ms, "kernel_ms_min": ev_ms[0],
                 "kernel_ms_median": ev_ms[len(ev_ms) // 2], "algorithmic_bytes": counts["bytes"],
                 "algorithmic_flops": counts["flops"], "tflops": tflops, "gbps": gbps})
    return roof


def library_gemm_tflops(n=8192, reps=10):
    """bf16 n x n x n product of the vendor library (hipBLASLt through torch), best and median of `reps` timed calls.
    Not a baseline of this op: it shows how far below the published matrix peak a plain GEMM runs on the same box, in
    the same process, minutes apart -- long MFMA-bound kernels are held by the power limit, and boxes differ."""
    import torch

    a = torch.randn(n, n, device="cuda:0", dtype=torch.bfloat16)
    b = torch.randn(n, n, device="cuda:0", dtype=torch.bfloat16)
    settle(lambda: a @ b)
    torch.cuda.synchronize()
    ts = []
    for _ in range(reps):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        a @ b
        e1.record()
        torch.cuda.synchronize()
        ts.append(e0.elapsed_time(e1))
    ts.sort()
    flops = 2.0 * n ** 3
    return {"n": n, "median": flops / ts[len(ts) // 2] / 1e9, "best": flops / ts[0] / 1e9}


def board_power_watts():
    """(power drawn now, power cap) of the first GPU from the driver's hwmon files, in watts; None where unreadable."""
    import glob

    def read(pattern):
        for f in sorted(glob.glob("/sys/class/drm/card*/device/hwmon/hwmon*/" + pattern)):
            try:
                return int(open(f).read()) / 1e6
            except (OSError, ValueError):
                pass
        return None

    now = read("power1_input")
    return (now if now is not None else read("power1_average")), read("power1_cap")


def sustain(fn, seconds, what, flops=None, nbytes=None, quiet=False):
    """Back-to-back launches of `fn` for `seconds`; the power sensor is read between batches of 50 launches."""
    import torch

    idle = board_power_watts()[0]
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    n, watts = 0, []
    while time.perf_counter() - t0 < seconds:
        for _ in range(50):
            fn()
        torch.cuda.synchronize()
        n += 50
        watts.append(board_power_watts()[0])
    ms = (time.perf_counter() - t0) / n * 1e3
    watts = sorted(w for w in watts if w is not None)
    res = {"sustain": what, "seconds": seconds, "launches": n, "ms_per_launch": ms, "power_idle_w": idle,
           "power_w_median": watts[len(watts) // 2] if watts else None, "power_cap_w": board_power_watts()[1]}
    if flops:
        res["tflops"] = flops / ms / 1e9
    if nbytes:
        res["gbps"] = nbytes / ms / 1e6
    if not quiet:
        print(json.dumps(res))
    return res


def graph_replay_ms(step, reps):
    """The call captured in a HIP graph and replayed `reps` times: milliseconds per replay (no host code per step)."""
    import torch

    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for _ in range(5):
        g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        g.replay()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / reps


def measure_ref_bench(steps, warmup, want_parity, want_baseline):
    """The reference's own benchmark grid (benchmarks/benchmark_ragged_page_attn.py:148-185: max_num_seqs {8, 16, 32} x
    page_size {8 .. 128}, 16 pages per sequence, 16 / 4 heads, head_dim 128, q_len ~ U[1, kv_len]), one entry per shape:
    microseconds per call and per HIP-graph replay (these batches are launch-latency bound), parity of every row against
    the CPU restatement of the reference program and that restatement's time for the whole batch on the host cores."""
    import torch

    from ejkernel_amd.modules import ragged_page_attention
    from ejkernel_amd.roofline import algorithmic_counts
    from ejkernel_amd.workloads import REF_BENCH_GRID, make_workload
    from oracle import rpa_oracle_c
    from tests.helpers import err_stats, oracle_args, to_np

    out_entries = []
    threads = rpa_oracle_c.max_threads()
    for S, page in REF_BENCH_GRID:
        name = f"ref_bench_{S}_{page}"
        batch = make_workload(name, device="cuda:0")
        m = batch.meta
        counts = algorithmic_counts(batch.q_lens, batch.kv_lens, num_q_heads=m["num_q_heads"], num_kv_heads=m["num_kv_heads"],
                                    head_dim=m["head_dim"], page_size=m["page_size"], sliding_window=None)

        def step():
            return ragged_page_attention(*batch.args(), **batch.kwargs())

        ms_per_step, ev_ms, out = time_steps(step, steps, warmup, settle_s=0.05)
        entry = {"workload": name, "max_num_seqs": S, "page_size": page, "query_tokens": counts["tokens"],
                 "kv_tokens": int(batch.kv_lens.sum()), "us_per_call": ms_per_step * 1e3,
                 "kernel_us_avg": sum(ev_ms) / len(ev_ms) * 1e3, "kernel_us_min": ev_ms[0] * 1e3,
                 "graph_replay_us": graph_replay_ms(step, max(steps, 50)) * 1e3,
                 "tokens_per_s": counts["tokens"] / (ms_per_step * 1e-3),
                 "gflops": counts["flops"] / 1e9, "mbytes": counts["bytes"] / 1e6}
        if want_parity or want_baseline:
            args = oracle_args(batch)
            t0 = time.perf_counter()
            ref = rpa_oracle_c.rpa_strict_c(*args, softmax_scale=batch.softmax_scale, io_dtype="bfloat16", threads=threads)
            dt = time.perf_counter() - t0
            rows = batch.total_valid_tokens
            if want_parity:
                mx, mean = err_stats(to_np(out), ref, rows)
                over = int((np_abs_diff(to_np(out)[:rows], ref[:rows]) > 2e-2).sum())
                entry["parity"] = {"max_abs": mx, "mean_abs": mean, "rows": rows, "elements_over_2e-2": over,
                                   "ok": bool(mx <= 2e-2 and mean <= 2e-3)}
            if want_baseline:
                entry["cpu_us_per_call"] = dt * 1e6
                entry["cpu_cores"] = int(threads)
        out_entries.append(entry)
        del batch, out
    torch.cuda.empty_cache()
    return out_entries


def np_abs_diff(a, b):
    import numpy as np

    return np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64))


def measure_config(name, steps, warmup, want_parity, queries_per_block=None):
    """One entry of "configs": the named workload at full size, timed like the headline one and checked against the
    CPU restatement on a small sample of its sequences.  `queries_per_block` is passed on as
    RaggedPageAttentionConfig.num_queries_per_block (the caller's hint for the kernel instantiation)."""
    import torch

    from ejkernel_amd.modules import RaggedPageAttentionConfig, ragged_page_attention
    from ejkernel_amd.roofline import algorithmic_counts
    from ejkernel_amd.workloads import make_workload

    batch = make_workload(name, device="cuda:0")
    cfg = None if queries_per_block is None else RaggedPageAttentionConfig(num_queries_per_block=queries_per_block)
    m = batch.meta
    counts = algorithmic_counts(batch.q_lens, batch.kv_lens, num_q_heads=m["num_q_heads"], num_kv_heads=m["num_kv_heads"],
                                head_dim=m["head_dim"], page_size=m["page_size"], sliding_window=batch.sliding_window)

    def step():
        return ragged_page_attention(*batch.args(), cfg=cfg, **batch.kwargs())

    ms_per_step, ev_ms, out = time_steps(step, steps, warmup)
    roof = roofline_of(counts, ev_ms)
    roof["traffic"] = measured_traffic_bytes(name)
    if roof["bound"] == "mfma" and not name.endswith("_padded"):
        roof["library_gemm_tflops"] = library_gemm_tflops()
    entry = {"workload": name, "ms_per_step": ms_per_step, "kernel_ms_avg": roof["kernel_ms_avg"],
             "tokens_per_s": counts["tokens"] / (ms_per_step * 1e-3), "roofline": roof,
             "host_overhead_ms": ms_per_step - roof["kernel_ms_avg"]}
    if name.endswith("_padded"):
        entry["static_shapes"] = {"total_tokens": int(batch.queries.shape[0]), "max_num_seqs": int(m["max_num_seqs"]),
                                  "num_seqs": len(batch.q_lens)}
        entry["num_queries_per_block"] = queries_per_block
    if name in ("decode_small", "prefill_chunk_after_8k", "chunk_beside_decodes"):
        # the launch-bound configurations: the same call replayed from a HIP graph, where no host code runs per step
        entry["graph_replay_ms"] = graph_replay_ms(step, max(steps, 50))
    if want_parity:
        if name in LONG_PROMPT_CONFIGS:
            entry["parity"] = long_prompt_parity(batch, out)
        else:
            entry["parity"] = cpu_sample_and_parity(batch, out, False, True, 0, budget_s=4.0)["parity"]
    del batch, out
    torch.cuda.empty_cache()
    return entry


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures one GPU only (the op shards without exchange by sequence or by "
              "kv head); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch

    from ejkernel_amd import _native
    from ejkernel_amd.modules import ragged_page_attention
    from ejkernel_amd.roofline import HBM_PEAK_GBPS, MFMA_BF16_PEAK_TFLOPS, algorithmic_counts
    from ejkernel_amd.workloads import WORKLOADS, make_workload

    _native.load()  # fail loudly before any timing if the HIP library is missing
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = "cuda:0"
    if args.op in ("page_attention", "ragged_decode"):
        return page_attention_main(args)
    if args.gemm_probe and args.sustain > 0:
        n = args.gemm_probe
        ga = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
        gb = torch.randn(n, n, device=dev, dtype=torch.bfloat16)
        return sustain(lambda: ga @ gb, args.sustain, f"library bf16 GEMM {n}^3", flops=2.0 * n ** 3)
    if args.gemm_probe:
        print(json.dumps({"gemm_probe": library_gemm_tflops(args.gemm_probe, max(args.steps, 3)), "unit": "TFLOP/s", "dtype": "bf16"}))
        return
    if args.copy_probe:
        n = args.copy_probe << 20
        src = torch.full((n,), 7, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            dst.copy_(src)
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.steps
        print(json.dumps({"copy_probe_bytes_read": n, "copy_probe_bytes_written": n, "steps": args.steps,
                          "ms_per_copy": dt * 1e3, "gbps_read_plus_write": 2 * n / dt / 1e9}))
        return
    batch = make_workload(args.workload, device=dev, scale=args.scale)
    m = batch.meta
    counts = algorithmic_counts(batch.q_lens, batch.kv_lens, num_q_heads=m["num_q_heads"],
                                num_kv_heads=m["num_kv_heads"], head_dim=m["head_dim"], page_size=m["page_size"],
                                sliding_window=batch.sliding_window)

    v3 = None
    if args.op == "rpa_v3":
        from ejkernel_amd.modules import ragged_page_attention_v3
        from ejkernel_amd.workloads import to_v3

        fp8 = args.cache_dtype == "fp8"
        v3 = to_v3(batch, seed=1, cache_dtype=torch.float8_e4m3fn if fp8 else None)
        if fp8:  # the algorithmic minimum reads every visible K/V row once, at one byte per element
            counts["bytes"] -= counts["kv_bytes"] // 2
            counts["kv_bytes"] //= 2
        # the new rows are read once and written once into the cache, on top of the attention traffic
        row_bytes = 2 * m["num_kv_heads"] * m["head_dim"] * (1 if fp8 else 2)
        counts["bytes"] += 2 * counts["tokens"] * row_bytes

    def step():
        if v3 is not None:
            return ragged_page_attention_v3(*v3.args(), **v3.kwargs())[0]
        return ragged_page_attention(*batch.args(), **batch.kwargs())

    if args.sustain > 0:
        return sustain(step, args.sustain, args.workload, flops=counts["flops"], nbytes=counts["bytes"])
    ms_per_step, ev_ms, out = time_steps(step, args.steps, args.warmup)
    kernel_ms = sum(ev_ms) / len(ev_ms)
    tokens = counts["tokens"]
    roof = roofline_of(counts, ev_ms)
    roof["traffic"] = measured_traffic_bytes(args.workload) if args.scale == 1.0 and v3 is None else None
    if roof["bound"] == "mfma" and args.scale == 1.0:
        roof["library_gemm_tflops"] = library_gemm_tflops()
    gbps, tflops = roof["gbps"], roof["tflops"]

    line = {
        "metric": "ragged paged-attn tokens/s" if v3 is None else "ragged paged-attn v3 (cache update + attention) tokens/s", "value": tokens / (ms_per_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "settle_s": SETTLE_S, "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {"workload": args.workload, "op": args.op, "description": WORKLOADS[args.workload], "scale": args.scale,
                   "query_tokens": tokens, "num_seqs": len(batch.q_lens), "kv_tokens": int(batch.kv_lens.sum())},
        "roofline": roof,
    }
    if not (args.no_cpu_baseline and args.no_parity):
        if v3 is None and args.workload in LONG_PROMPT_CONFIGS and args.scale == 1.0:
            if not args.no_parity:
                line["parity"] = long_prompt_parity(batch, out)
        elif v3 is None:
            line.update(cpu_sample_and_parity(batch, out, not args.no_cpu_baseline, not args.no_parity, args.cpu_seqs))
        else:
            # Repeating the call rewrites the same rows with the same values, so the cache after the timed steps is the
            # cache after one update; the oracle starts from the pages with the new rows still holding their old content,
            # which only differ at the positions it overwrites itself.
            line.update(cpu_sample_and_parity_v3(batch, v3, out, not args.no_cpu_baseline, not args.no_parity,
                                                 args.cpu_seqs))
    if (not args.no_configs and args.workload == "decode_llama3_8b" and args.op == "rpa" and args.scale == 1.0):
        del batch, out
        torch.cuda.empty_cache()
        # A failure in one of the other configurations must not cost the headline line: it is reported in place of the
        # entry (the exception's text; nothing is retried, and a device fault would end the process anyway).
        line["configs"] = []
        for item in EXTRA_CONFIGS:
            name, hint = item if isinstance(item, tuple) else (item, None)
            try:
                line["configs"].append(measure_config(name, args.steps, args.warmup, not args.no_parity, hint))
            except Exception as e:  # noqa: BLE001
                line["configs"].append({"workload": name, "error": f"{type(e).__name__}: {e}"[:500]})
                torch.cuda.empty_cache()
        try:
            line["ref_bench"] = measure_ref_bench(args.steps, args.warmup, not args.no_parity, not args.no_cpu_baseline)
        except Exception as e:  # noqa: BLE001
            line["ref_bench"] = {"error": f"{type(e).__name__}: {e}"[:500]}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
