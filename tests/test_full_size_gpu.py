"""The five benchmark workloads (and the prefill half of the mixed one, which runs on the pipelined tiles) at their full
sizes on the device.

At these sizes the whole batch cannot go through the CPU oracle in seconds, so each workload is checked
(a) on a seeded sample of its sequences against the C restatement of the reference (same tolerance as the
small cases: max-abs <= 2e-2, mean-abs <= 2e-3; rows where the reference program yields NaN -- a leading KV
block entirely left of the sliding window -- are compared with the float64 evaluation), and (b) through
properties that do not depend on size: finite output, zero rows past the batch, bitwise invariance under a
permutation of the physical pages, bitwise reproducibility, and agreement of every decode row with the same
sequence run alone (identical up to the fp32 rounding of a different split, i.e. a last-place bf16 flip).
"""

import numpy as np
import pytest
import torch

from ejkernel_amd.modules import ragged_page_attention
from ejkernel_amd.workloads import Batch, compact_for_host, make_workload
from oracle import rpa_oracle_c
from tests.helpers import (BF16_MAX_ABS, BF16_MEAN_ABS, assert_bf16_parity_stepwise, err_stats, oracle_args, run_exact,
                           to_np)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run(b):
    out = ragged_page_attention(*b.args(), **b.kwargs())
    torch.cuda.synchronize()
    return out


def check_sample(b, out, n_seqs, seed=0):
    rng = np.random.default_rng(seed)
    order = [int(s) for s in rng.permutation(len(b.q_lens))]
    if b.sliding_window:
        # The reference program turns a row NaN when one of its 64-page KV blocks lies entirely left of the row's window,
        # and such rows can only be held against the float64 evaluation.  Half of the sample is therefore taken from
        # the sequences short enough to have no such block, so that the restatement of the program itself is what
        # checks a windowed workload too.
        short = [s for s in order if b.kv_lens[s] < b.sliding_window + 64 * b.meta["page_size"]]
        head = short[: n_seqs // 2]
        order = head + [s for s in order if s not in head]
    longest = int(np.argmax(b.q_lens))   # a workload's one long chunk, if it has one, is always in the sample
    if b.q_lens[longest] > 1:
        order = [longest] + [s for s in order if s != longest]
    ids = sorted(order[:n_seqs])
    sub = compact_for_host(b, ids)
    ref = rpa_oracle_c.rpa_strict_c(*oracle_args(sub), softmax_scale=sub.softmax_scale,
                                    logits_soft_cap=sub.logits_soft_cap, sliding_window=sub.sliding_window)
    rows = sub.total_valid_tokens
    nan_rows = np.isnan(ref[:rows]).any(axis=(1, 2))
    if nan_rows.any():
        ref[:rows][nan_rows] = run_exact(sub)[:rows][nan_rows]
    got = to_np(out[sub.meta["rows"].to(out.device)])
    mx, mean = err_stats(got, ref, rows)
    assert mx <= BF16_MAX_ABS and mean <= BF16_MEAN_ABS, (b.name, mx, mean)
    if b.sliding_window and any(b.kv_lens[s] < b.sliding_window + 64 * b.meta["page_size"] for s in ids):
        assert nan_rows.sum() < rows, "no row of the sample was checked against the restatement of the program"
    return sub, int(nan_rows.sum())


def permuted(b, seed=9):
    P = b.kv_pages.shape[0]
    perm = torch.randperm(P, generator=torch.Generator().manual_seed(seed)).to(DEV)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(P, device=DEV)
    b2 = Batch(**{**b.__dict__})
    b2.kv_pages = b.kv_pages[perm]
    b2.block_tables = inv[b.block_tables.long()].to(torch.int32)
    return b2


@pytest.mark.parametrize("name,n_sample,permute", [("decode_small", 8, True), ("decode_llama3_8b", 12, True),
                                                   ("mixed_prefill_decode", 14, True), ("mixed_prefill_only", 3, True),
                                                   ("gemma2_local", 8, False), ("decode_long_context", 5, False),
                                                   ("decode_head_dim_96", 12, True), ("mixed_head_dim_96", 10, True),
                                                   ("prefill_head_dim_256", 1, True), ("decode_head_dim_64", 12, True),
                                                   ("prefill_chunk_after_8k", 1, True), ("chunk_beside_decodes", 6, True)])
def test_full_size_workload(name, n_sample, permute):
    b = make_workload(name, device=DEV)
    out = run(b)
    total = b.total_valid_tokens
    assert torch.isfinite(out.float()).all()
    assert not out[total:].any()
    assert torch.equal(run(b), out)  # reproducible bit for bit
    sub, _ = check_sample(b, out, n_sample)
    if permute:
        assert torch.equal(run(permuted(b)), out)
    # one sampled sequence on its own: same rows up to a last-place flip
    s = int(np.argmax(b.q_lens == b.q_lens.min()))
    alone = compact_for_host(b, [s])
    dev = Batch(**{**alone.__dict__})
    for f in ("queries", "kv_pages", "context_lens", "block_tables", "query_start_loc", "num_seqs"):
        setattr(dev, f, getattr(alone, f).to(DEV))
    got = run(dev)[: int(b.q_lens[s])].float()
    cu = b.query_start_loc.cpu().numpy()
    want = out[cu[s]:cu[s + 1]].float()
    assert (got - want).abs().max().item() <= 2.0 ** -7 * max(1.0, want.abs().max().item())
    del b, out
    torch.cuda.empty_cache()


@pytest.mark.parametrize("name,hint,n_sample", [("decode_llama3_8b", 16, 12), ("mixed_prefill_decode", 128, 14),
                                                ("mixed_prefill_only", 256, 3)])
def test_padded_static_shapes_with_and_without_the_config_hint(name, hint, n_sample):
    """The same sequences, pages and queries inside the static shapes of a serving caller (max_num_seqs 512, query rows
    rounded up to 8192 / 16384, num_seqs as is).  With RaggedPageAttentionConfig.num_queries_per_block naming the tile
    shape the padded call runs the instantiation the unpadded call gets by default: the rows of the batch are bitwise
    those.  Without the hint the library goes by the padded shapes (another instantiation for two of the three): the
    sample must still meet the parity bound.  Either way every row past the batch is zero."""
    from ejkernel_amd.modules import RaggedPageAttentionConfig

    base = make_workload(name, device=DEV)
    want = run(base)
    total = base.total_valid_tokens
    del base
    torch.cuda.empty_cache()
    b = make_workload(name + "_padded", device=DEV)
    assert b.block_tables.shape[0] == 512 and b.queries.shape[0] in (8192, 16384) and b.total_valid_tokens == total
    hinted = ragged_page_attention(*b.args(), cfg=RaggedPageAttentionConfig(num_queries_per_block=hint), **b.kwargs())
    torch.cuda.synchronize()
    assert torch.equal(hinted[:total], want[:total])
    assert not hinted[total:].any()
    plain = run(b)
    assert torch.isfinite(plain.float()).all() and not plain[total:].any()
    check_sample(b, plain, n_sample)
    check_sample(b, hinted, n_sample)
    del b, want, hinted, plain
    torch.cuda.empty_cache()


@pytest.mark.parametrize("S,page", [(8, 8), (8, 128), (16, 16), (16, 64), (32, 8), (32, 32), (32, 128)])
def test_reference_benchmark_grid_shapes(S, page):
    """Shapes of the reference's own benchmark (max_num_seqs x page_size at 16 pages per sequence, 16 / 4 heads,
    q_len ~ U[1, kv_len], identity block table): every row against the C restatement, on the library's choice of
    instantiation and on the forced prefill tiles."""
    from ejkernel_amd.modules import RaggedPageAttentionConfig

    b = make_workload(f"ref_bench_{S}_{page}", device=DEV)
    ref = rpa_oracle_c.rpa_strict_c(*oracle_args(b), softmax_scale=b.softmax_scale)
    rows = b.total_valid_tokens
    for hint in (None, 16, 128, 256):
        out = ragged_page_attention(*b.args(), cfg=RaggedPageAttentionConfig(num_queries_per_block=hint), **b.kwargs())
        torch.cuda.synchronize()
        assert_bf16_parity_stepwise(to_np(out)[:rows], ref[:rows], f"ref_bench {S} x page {page}, hint {hint}")
        assert not out[rows:].any()


def test_tile_kernel_is_picked_on_the_device_where_the_host_cannot_tell():
    """Static shapes that say nothing about the batch (many rows, few tokens per max_num_seqs, no flag, no hint): both
    tile kernels are enqueued and the device picks one from the lengths.  A batch whose prefill work outweighs its
    decode stream must come out bit for bit as the pipelined tiles give it, one whose stream outweighs the chunks as
    the 128-row tiles do, and so must one of short chunks (fewer than 512 keys per query row on average: a pipelined
    tile's fixed costs are hidden by nothing); and the pair of launches replays from a HIP graph on new queries."""
    from ejkernel_amd import _native
    from ejkernel_amd.modules.operations import RaggedPageAttention, RaggedPageAttentionConfig
    from ejkernel_amd.workloads import make_batch

    def run_flags(bb, flags, out=None):
        o = RaggedPageAttention().run(*bb.args(), softmax_scale=bb.softmax_scale, cfg=RaggedPageAttentionConfig(), _flags=flags,
                                      _out=out)
        torch.cuda.synchronize()
        return o

    rng = np.random.default_rng(3)
    chunks = make_batch([600] * 4 + [1] * 8, [900] * 4 + list(rng.integers(1000, 3000, size=8)), num_q_heads=32,
                        num_kv_heads=8, head_dim=128, page_size=32, pages_per_seq=128, seed=51, device=DEV, max_num_seqs=64)
    stream = make_batch([600] + [1] * 60, [900] + list(rng.integers(3000, 4096, size=60)), num_q_heads=32, num_kv_heads=8,
                        head_dim=128, page_size=32, pages_per_seq=128, seed=52, device=DEV, max_num_seqs=64)
    short = make_batch([200] * 16, [200] * 12 + [500] * 4, num_q_heads=32, num_kv_heads=8, head_dim=128, page_size=32,
                       pages_per_seq=128, seed=53, device=DEV, max_num_seqs=64)
    pipe, plain = _native.RPA_FLAG_PIPE_TILES, _native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES
    for b, picked, other in ((chunks, pipe, plain), (stream, plain, pipe), (short, plain, pipe)):
        assert b.queries.shape[0] * 32 > 20480 and b.queries.shape[0] < 128 * 64   # no rule of the host's applies
        out = run_flags(b, 0)
        assert torch.equal(out, run_flags(b, picked))
        assert not torch.equal(out, run_flags(b, other))   # (the other kernel's rounding differs somewhere)
        sub, _ = check_sample(b, out, 4)
        assert not out[b.total_valid_tokens:].any()
    # the two launches of one call in a HIP graph
    b = chunks
    out = torch.zeros_like(b.queries)
    run_flags(b, 0, out)
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            RaggedPageAttention().run(*b.args(), softmax_scale=b.softmax_scale, cfg=RaggedPageAttentionConfig(), _out=out)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    gen = torch.Generator(device=DEV).manual_seed(9)
    for k in range(3):
        b.queries[: b.total_valid_tokens] = torch.randn(b.total_valid_tokens, 32, 128, device=DEV, generator=gen).to(torch.bfloat16)
        out.fill_(5.0)
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.clone(), run_flags(b, pipe)), f"replay {k}"


def test_long_prompts_on_pipelined_and_plain_tiles():
    """prefill_long (2 prompts x 8192 tokens) is too much for the CPU restatement in seconds (its scaled form is checked
    against it elsewhere): here the two tile kernels must agree with each other within the parity bound, each must be
    reproducible bit for bit and invariant under a permutation of the physical pages, and nothing past the batch may be
    written."""
    from ejkernel_amd import _native
    from ejkernel_amd.modules.operations import RaggedPageAttention, RaggedPageAttentionConfig

    b = make_workload("prefill_long", device=DEV)

    def run_flags(bb, flags):
        o = RaggedPageAttention().run(*bb.args(), softmax_scale=bb.softmax_scale, cfg=RaggedPageAttentionConfig(), _flags=flags)
        torch.cuda.synchronize()
        return o

    pipe = run_flags(b, _native.RPA_FLAG_PIPE_TILES)
    plain = run_flags(b, _native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES)
    assert torch.equal(run(b), pipe)  # the default for this batch is the pipelined tile
    assert torch.isfinite(pipe.float()).all() and torch.isfinite(plain.float()).all()
    assert not pipe[b.total_valid_tokens:].any()
    diff = (pipe.float() - plain.float()).abs()
    assert diff.max().item() <= BF16_MAX_ABS and diff.mean().item() <= BF16_MEAN_ABS, (diff.max().item(), diff.mean().item())
    assert torch.equal(run_flags(b, _native.RPA_FLAG_PIPE_TILES), pipe)
    assert torch.equal(run_flags(permuted(b), _native.RPA_FLAG_PIPE_TILES), pipe)
