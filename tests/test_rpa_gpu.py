"""Parity of the HIP path (called through the C ABI) against the CPU oracle.

bf16: max-abs <= 2e-2 and mean-abs <= 2e-3 against ``rpa_strict`` (the restatement of the
reference's XLA implementation, bf16 rounding points included).  fp32 mode: <= 1e-5 against
the float64 evaluation; page gathering is checked bit-exactly on cases with a closed form.
"""

import numpy as np
import pytest
import torch

from ejkernel_amd import _native
from ejkernel_amd.modules import RaggedPageAttention, RaggedPageAttentionConfig, ragged_page_attention
from ejkernel_amd.workloads import Batch, compact_for_host, make_batch, make_workload
from tests.helpers import (F32_MAX_ABS, assert_bf16_parity, assert_bf16_parity_stepwise, err_stats, random_rpa_batch, random_serving_batch,
                           run_exact, run_strict, to_np, two_key_cap_batch)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

# the MFMA kernel as the library picks it (small batches: without prefill tiles), the MFMA kernel with prefill tiles
# forced, and the scalar kernel
PATHS = [pytest.param(0, id="tiled"),
         pytest.param(_native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES, id="tiles"),
         pytest.param(_native.RPA_FLAG_PIPE_TILES, id="pipe"),  # head_dim 128, pages of 16 keys or more; else as "tiles"
         pytest.param(_native.RPA_FLAG_FORCE_GENERIC, id="generic")]


def run_hip(b: Batch, flags=0, compute_dtype=None, softmax_aux=None, cfg=None):
    if compute_dtype is None:
        compute_dtype = b.queries.dtype
    aux = None if softmax_aux is None else torch.as_tensor(softmax_aux, device=b.queries.device)
    out = RaggedPageAttention().run(*b.args(), softmax_scale=b.softmax_scale, logits_soft_cap=b.logits_soft_cap,
                                    compute_dtype=compute_dtype, sliding_window=b.sliding_window, softmax_aux=aux,
                                    cfg=cfg or RaggedPageAttentionConfig(), _flags=flags)
    torch.cuda.synchronize()
    return out


def small(q_lens, kv_lens, **kw):
    args = dict(num_q_heads=8, num_kv_heads=2, head_dim=128, page_size=16, pages_per_seq=16, seed=7, device=DEV)
    args.update(kw)
    return make_batch(q_lens, kv_lens, **args)


# ----------------------------------------------------------------------------- fp32 mode: gather exactness


@pytest.mark.parametrize("flags", PATHS)
def test_fp32_mode_matches_float64_evaluation(flags):
    b = make_workload("decode_small", device=DEV, dtype=torch.float32)
    out = to_np(run_hip(b, flags, compute_dtype=torch.float32))
    rows = b.total_valid_tokens
    mx, _ = err_stats(out, run_exact(b), rows)
    assert mx <= F32_MAX_ABS, mx
    assert not out[rows:].any()


@pytest.mark.parametrize("flags", PATHS)
def test_fp32_mode_ragged_mix(flags):
    b = small([9, 1, 0, 17, 2, 4], [40, 250, 8, 17, 133, 256], dtype=torch.float32, max_num_seqs=8)
    out = to_np(run_hip(b, flags, compute_dtype=torch.float32))
    mx, _ = err_stats(out, run_exact(b), b.total_valid_tokens)
    assert mx <= F32_MAX_ABS, mx


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_single_key_gather_is_bit_exact(flags, dtype):
    """kv_len = 1 => out == the V row of token 0, bit for bit (page, slot and head indexing)."""
    S = 12
    b = small(np.ones(S, int), np.ones(S, int), dtype=dtype, num_q_heads=8, num_kv_heads=4)
    out = run_hip(b, flags)
    bt = b.block_tables.long()
    want = b.kv_pages[bt[:, 0], 0, 1::2, :].repeat_interleave(2, dim=1)  # [S, Hq, D]
    assert torch.equal(out[:S], want)


@pytest.mark.parametrize("flags", PATHS)
def test_zero_query_mean_of_values_fp32(flags):
    """q = 0 => out = mean of the visible V rows; V carries small integers so fp32 sums are exact."""
    b = small([3, 1, 5], [37, 200, 5], dtype=torch.float32, num_q_heads=4, num_kv_heads=2, head_dim=64)
    b.queries.zero_()
    gen = torch.Generator(device=DEV).manual_seed(1)
    b.kv_pages.copy_(torch.randint(-8, 9, b.kv_pages.shape, generator=gen, device=DEV).float())
    out = to_np(run_hip(b, flags, compute_dtype=torch.float32))
    mx, _ = err_stats(out, run_exact(b), b.total_valid_tokens)
    assert mx <= 2e-6, mx


# ----------------------------------------------------------------------------- bf16 parity vs the strict oracle


@pytest.mark.parametrize("flags", PATHS)
def test_bf16_decode_small_full_size(flags):
    b = make_workload("decode_small", device=DEV)
    out = to_np(run_hip(b, flags))
    assert_bf16_parity(out, run_strict(b), b.total_valid_tokens, "decode_small")
    assert not out[b.total_valid_tokens:].any()


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("name,scale", [("decode_llama3_8b", 0.06), ("mixed_prefill_decode", 0.08),
                                        ("decode_long_context", 0.04), ("prefill_long", 0.08), ("prefill_head_dim_64", 0.12),
                                        ("decode_head_dim_64", 0.06)])
def test_bf16_scaled_workloads(flags, name, scale):
    b = make_workload(name, device=DEV, scale=scale)
    out = to_np(run_hip(b, flags))
    assert_bf16_parity(out, run_strict(b), b.total_valid_tokens, name)


@pytest.mark.parametrize("flags", PATHS)
def test_bf16_gemma2_local_scaled(flags):
    """Window + soft cap + head_dim 256.  Where the strict oracle turns NaN (a leading KV block entirely outside
    the window) the row is compared with the float64 evaluation instead."""
    b = make_workload("gemma2_local", device=DEV, scale=0.1)
    out = to_np(run_hip(b, flags))
    rows = b.total_valid_tokens
    strict, exact = run_strict(b), run_exact(b)
    nan_rows = np.isnan(strict[:rows]).any(axis=(1, 2))
    ref = np.where(nan_rows[:, None, None], exact[:rows], strict[:rows])
    assert_bf16_parity(out, ref, rows, "gemma2_local")


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("hq,hkv", [(4, 4), (8, 4), (8, 2), (16, 2), (8, 1)])
def test_bf16_gqa_ratios(flags, hq, hkv):
    b = small([6, 1, 1, 33], [70, 255, 256, 33], num_q_heads=hq, num_kv_heads=hkv)
    assert_bf16_parity(to_np(run_hip(b, flags)), run_strict(b), b.total_valid_tokens, f"gqa {hq}/{hkv}")


@pytest.mark.parametrize("D", [128, 256, 64])
@pytest.mark.parametrize("hq,hkv,q_len", [(2, 2, 1), (8, 4, 1), (8, 2, 1), (16, 2, 1), (16, 2, 2), (12, 4, 1), (8, 2, 3)])
def test_bf16_few_long_sequences_split_into_many_parts(hq, hkv, q_len, D):
    """One or two long sequences on the whole grid: every (sequence, kv head) is cut into dozens of parts, which the
    last wavefront to arrive merges several at a time on the lanes of the rows a decode tile does not have (1, 2, 4,
    8 or 16 rows per tile here, 3 and 6 padded to 4 and 8).  Parity, and the same bits on every call.
    With so few (sequence, kv head)s the stream is cut by workgroup up to head_dim 128 (four wavefronts a quarter of
    the workgroup's share each, merged in LDS, then the split through memory over a quarter of the parts); a
    `num_kv_pages_per_block` names the cut and gives the one by wavefront, which must agree."""
    b = small([q_len, q_len], [8192, 5000], num_q_heads=hq, num_kv_heads=hkv, pages_per_seq=512, head_dim=D)
    out = run_hip(b)
    assert_bf16_parity(to_np(out), run_strict(b), b.total_valid_tokens, f"{hq}/{hkv} q_len {q_len} D {D}")
    for _ in range(3):
        assert torch.equal(run_hip(b), out)
    by_wave = run_hip(b, cfg=RaggedPageAttentionConfig(num_kv_pages_per_block=8))
    assert_bf16_parity(to_np(by_wave), run_strict(b), b.total_valid_tokens, "cut by wavefront")
    assert (out.float() - by_wave.float()).abs().max().item() <= 2e-2
    assert_bf16_parity(to_np(run_hip(b, _native.RPA_FLAG_PREFILL_TILES)), run_strict(b), b.total_valid_tokens, "tiles")


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("page", [1, 4, 8, 16, 32, 64, 128])
def test_bf16_page_sizes(flags, page):
    pps = max(2, 512 // page)
    b = small([5, 1, 1, 40], [300, 511, 17, 40], page_size=page, pages_per_seq=pps)
    assert_bf16_parity(to_np(run_hip(b, flags)), run_strict(b), b.total_valid_tokens, f"page {page}")


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("D", [64, 128, 256])
def test_bf16_head_dims(flags, D):
    b = small([5, 1, 2, 40], [300, 511, 17, 40], head_dim=D, pages_per_seq=32)
    assert_bf16_parity(to_np(run_hip(b, flags)), run_strict(b), b.total_valid_tokens, f"D {D}")


@pytest.mark.parametrize("hq,hkv", [(8, 2), (4, 4), (32, 4), (64, 8), (6, 3), (32, 2), (16, 8)])
@pytest.mark.parametrize("window,cap,sinks", [(None, None, False), (40, 20.0, True)])
def test_bf16_head_dim_64_two_kv_heads_per_item(hq, hkv, window, cap, sinks):
    """head_dim 64 in the wave-level loop: with an even number of kv heads and at most 8 query heads per kv head, an
    item covers two kv heads (their rows share a 16-row tile: 2, 8 or 16 rows per decode token here; 3 kv heads and 16
    query heads per kv head keep one kv head per item).  Decode tokens, short chunks whose row tiles straddle tokens and
    heads, a sequence without keys before its own token, split (sequence, head pair)s; the exact kernel as cross-check."""
    b = small([1, 3, 1, 7, 1, 2], [300, 90, 1, 7, 511, 40], num_q_heads=hq, num_kv_heads=hkv, head_dim=64, pages_per_seq=32,
              sliding_window=window, logits_soft_cap=cap)
    aux = (torch.randn(hq, 2, generator=torch.Generator().manual_seed(5)) * 2).numpy() if sinks else None
    ref = run_strict(b, softmax_aux=aux)
    out = run_hip(b, softmax_aux=aux)
    assert_bf16_parity(to_np(out), ref, b.total_valid_tokens, f"{hq}/{hkv} W={window} cap={cap} sinks={sinks}")
    assert torch.equal(run_hip(b, softmax_aux=aux), out)
    assert_bf16_parity(to_np(run_hip(b, _native.RPA_FLAG_FORCE_GENERIC, softmax_aux=aux)), ref, b.total_valid_tokens, "generic")
    # one long sequence: every head pair is cut into many parts and merged
    if window is None:
        b = small([1], [8000], num_q_heads=hq, num_kv_heads=hkv, head_dim=64, pages_per_seq=512)
        assert_bf16_parity(to_np(run_hip(b)), run_strict(b), 1, f"long {hq}/{hkv}")
    # pages shorter than a 16-token sub-tile (per-lane page look-up) and longer ones
    for page in (4, 64):
        # (the reference yields NaN where one of its 64-page KV blocks lies left of the window: no window on 4-token pages)
        b = small([1, 2, 1], [301, 77, 130], num_q_heads=hq, num_kv_heads=hkv, head_dim=64, page_size=page,
                  pages_per_seq=max(2, 512 // page), sliding_window=window if page == 64 else None, logits_soft_cap=cap)
        assert_bf16_parity(to_np(run_hip(b)), run_strict(b), b.total_valid_tokens, f"page {page} {hq}/{hkv}")


@pytest.mark.parametrize("hq,hkv,D", [(8, 2, 128), (32, 8, 128), (4, 4, 128), (16, 1, 128), (8, 2, 64), (16, 8, 64), (6, 3, 64)])
@pytest.mark.parametrize("window,cap,sinks", [(None, None, False), (40, 20.0, True), (300, None, False)])
def test_bf16_small_decode_batches_one_workgroup_per_kv_head(hq, hkv, D, window, cap, sinks):
    """A decode batch of few short sequences runs one workgroup per (sequence, kv head): each of its four wavefronts
    walks a quarter of the keys and the partial states are merged in LDS.  Lengths around the tile and quarter
    boundaries (wavefronts without keys, a last tile of one key) up to 512 keys; up to 1024 in a batch of 32
    (sequence, kv head)s or more, where the longer limit applies; and the first batch again with a chunk of three
    tokens and a sequence of one key in it (with more than 16 rows the chunk is a wave-level item and sends the whole
    batch the usual way; with fewer it is one more row tile of the mode, whose rows belong to three tokens).
    `num_kv_pages_per_block` names the split and switches the mode off: the split over the grid, with its merge
    through memory, must agree with it and with the oracle."""
    aux = (torch.randn(hq, 2, generator=torch.Generator().manual_seed(5)) * 2).numpy() if sinks else None
    lens = [1, 31, 32, 33, 64, 65, 96, 97, 100, 128, 129, 255, 300, 500, 512]
    cases = [([1] * 15, lens, 32), ([1] * 15 + [3, 1], lens + [7, 1], 32)]
    n_more = -(-32 // hkv) + 1   # enough sequences for 32 (sequence, kv head)s
    rng = np.random.default_rng(11)
    cases.append(([1] * n_more, [1024, 1000, 513] + rng.integers(1, 1025, size=n_more - 3).tolist(), 64))
    if hkv == 8:   # more (sequence, kv head)s than streaming workgroups: 480 of the grid's 512 workgroups, and all of them
        cases.append(([1] * 60, rng.integers(1, 700, size=60).tolist(), 64))
        cases.append(([1] * 64, rng.integers(1, 300, size=64).tolist(), 32))
    for ql, kl, pps in cases:
        b = small(ql, kl, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, pages_per_seq=pps, sliding_window=window,
                  logits_soft_cap=cap, seed=23)
        ref = run_strict(b, softmax_aux=aux)
        out = run_hip(b, softmax_aux=aux)
        rows = b.total_valid_tokens
        assert_bf16_parity(to_np(out), ref, rows, f"{hq}/{hkv} D={D} W={window} cap={cap} sinks={sinks}")
        assert torch.equal(run_hip(b, softmax_aux=aux), out)   # deterministic
        assert not out[rows:].any()
        split = run_hip(b, softmax_aux=aux, cfg=RaggedPageAttentionConfig(num_kv_pages_per_block=4))
        assert_bf16_parity(to_np(split), ref, rows, "split over the grid")
        # the two ways of cutting a row's keys differ by fp32 summation order only: a bf16 step or two of the largest outputs
        assert (out[:rows].float() - split[:rows].float()).abs().max().item() <= 2e-2


@pytest.mark.parametrize("hq,hkv,D", [(32, 8, 128), (8, 2, 128), (16, 2, 256), (16, 2, 64), (12, 4, 96)])
@pytest.mark.parametrize("window,cap,sinks", [(None, None, False), (1500, 30.0, True)])
def test_bf16_few_long_chunks_have_their_key_ranges_cut(hq, hkv, D, window, cap, sinks):
    """One or two long chunks after a long context are few 128-row tiles for the grid's 512 workgroups: the library
    takes the 128-row tile kernel for such shapes and the device cuts every tile's key range into up to four runs, a
    workgroup each, whose states (reference point, sum, unnormalised output) meet in the workspace where the last one
    to arrive adds them up in run order.  Parity with the oracle, the same bits on every call, agreement with the
    wave-level loop (`num_queries_per_block=16`, which never cuts), zeros past the batch; chunks whose tiles differ
    in length (the first one sees 1 key tile or 30), a chunk that ends inside a tile, an empty run (the cut leaves
    the last runs of a short range without keys)."""
    aux = (torch.randn(hq, 2, generator=torch.Generator().manual_seed(5)) * 2).numpy() if sinks else None
    # (the last one: a chunk beside decode steps -- the tiles' parts then share the workspace with the decode stream's
    # partial states, which the long decode sequence makes sure there are)
    cases = [([300], [2300]), ([257, 40], [1900, 700]), ([512], [512]), ([64], [3000]), ([280, 1, 1, 1], [2000, 3000, 17, 900])]
    for ql, kl in cases:
        b = small(ql, kl, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, pages_per_seq=192, sliding_window=window,
                  logits_soft_cap=cap, seed=29)
        ref = run_strict(b, softmax_aux=aux)
        rows = b.total_valid_tokens
        nan_rows = np.isnan(ref[:rows]).any(axis=(1, 2))   # the reference program's window defect: float64 stands in
        if nan_rows.any():
            ref[:rows][nan_rows] = run_exact(b, softmax_aux=aux)[:rows][nan_rows]
        for flags in (0, _native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES):
            out = run_hip(b, flags, softmax_aux=aux)
            assert_bf16_parity(to_np(out), ref, rows, f"{ql}/{kl} {hq}/{hkv} D={D} W={window} flags={flags}")
            assert torch.equal(run_hip(b, flags, softmax_aux=aux), out)
            assert not out[rows:].any()
        by_wave = run_hip(b, softmax_aux=aux, cfg=RaggedPageAttentionConfig(num_queries_per_block=16))
        assert (out[:rows].float() - by_wave[:rows].float()).abs().max().item() <= 2e-2 * max(1.0, by_wave[:rows].float().abs().max().item())


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("hq,hkv,D", [(16, 2, 256), (8, 2, 256), (8, 2, 128), (32, 8, 128), (8, 2, 64), (4, 4, 64)])
@pytest.mark.parametrize("window", [None, 48])
def test_bf16_prefill_tiles_over_many_key_tiles(flags, hq, hkv, D, window):
    """Prefill chunks whose workgroup tiles walk three and more K/V tiles (the LDS stages are refilled while in
    use), with and without earlier context, a partial last row tile, and decode sequences in the same batch."""
    b = small([200, 1, 70, 130, 3], [200, 300, 100, 400, 90], num_q_heads=hq, num_kv_heads=hkv, head_dim=D,
              pages_per_seq=32, sliding_window=window)
    out = to_np(run_hip(b, flags))
    assert_bf16_parity(out, run_strict(b), b.total_valid_tokens, f"prefill tiles {hq}/{hkv} D={D} W={window}")


@pytest.mark.parametrize("page", [4, 8, 16, 64])
@pytest.mark.parametrize("hq,hkv", [(8, 2), (16, 2), (6, 2)])
@pytest.mark.parametrize("window,sinks", [(None, False), (48, True)])
def test_bf16_head_dim_64_prefill_tiles(page, hq, hkv, window, sinks):
    """head_dim 64 has prefill tiles of its own: 256 rows per workgroup, 128-byte K/V rows (two rows per LDS bank
    line, eight rows per fetch block -- more than a page of four tokens holds).  Chunks of one partial tile, of two
    and of five tiles, with and without earlier context, a window and sinks (the attention shape of gpt-oss)."""
    pps = -(-576 // page)
    pps = pps if pps < 64 else -(-pps // 64) * 64   # the reference's block-table windows clamp in rows of other lengths
    b = small([300, 1, 70, 130, 3], [300, 300, 100, 517, 90], num_q_heads=hq, num_kv_heads=hkv, head_dim=64,
              page_size=page, pages_per_seq=pps, sliding_window=window)
    aux = None
    if sinks:
        aux = torch.from_numpy(np.random.default_rng(4).standard_normal((hq, 1)).astype(np.float32)).to(torch.bfloat16)
    out = to_np(run_hip(b, _native.RPA_FLAG_PREFILL_TILES, softmax_aux=None if aux is None else aux.to(DEV)))
    aux_np = None if aux is None else aux.float().numpy()
    rows, what = b.total_valid_tokens, f"D=64 tiles page {page} {hq}/{hkv} W={window} sinks={sinks}"
    strict, exact = run_strict(b, softmax_aux=aux_np, aux_dtype="bfloat16")[:rows], run_exact(b, softmax_aux=aux_np)[:rows]
    finite = np.isfinite(strict).all(axis=(1, 2))  # short pages: the restatement's first KV block under a window is NaN
    assert finite.mean() > 0.5
    assert_bf16_parity_stepwise(out[:rows][finite], strict[finite], what)
    mx, mean = err_stats(out, exact, rows)
    assert mx <= 4e-2 and mean <= 2e-3, f"{what}: vs float64 max-abs {mx:.4g} mean-abs {mean:.4g}"


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("window,cap", [(None, None), (48, 20.0)])
def test_bf16_fp32_logit_arithmetic_on_prefill_tiles(D, window, cap):
    """RPA_FLAG_FP32_LOGITS (the arithmetic of ragged_page_attention_v3: the query enters unscaled, the fp32 logits
    take the scale) on the prefill tiles of every head_dim, against the float64 evaluation: what is left is the bf16
    rounding of the probabilities and of the output."""
    b = small([300, 1, 70, 130, 3], [300, 300, 100, 517, 90], num_q_heads=8, num_kv_heads=2, head_dim=D,
              page_size=16, pages_per_seq=36, sliding_window=window, logits_soft_cap=cap)
    exact = run_exact(b)
    for tiles in (_native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES, _native.RPA_FLAG_PIPE_TILES):
        out = to_np(run_hip(b, tiles | _native.RPA_FLAG_FP32_LOGITS))
        mx, mean = err_stats(out, exact, b.total_valid_tokens)
        assert np.isfinite(out).all() and mx <= 2e-2 and mean <= 1e-3, \
            f"D={D} W={window} cap={cap} tiles={tiles}: max-abs {mx:.4g} mean-abs {mean:.4g}"


@pytest.mark.parametrize("hq,hkv,D", [(8, 2, 128), (16, 2, 256), (8, 2, 64)])
@pytest.mark.parametrize("window", [None, 48])
def test_bf16_long_chunks_in_a_decode_shaped_batch(hq, hkv, D, window):
    """A small batch runs on the kernel without prefill tiles: chunks with many row tiles are then walked as wave-level
    items (the default path of most cases in this file; here with more sequence slots than sequences)."""
    b = small([40, 1, 1, 23, 1], [300, 300, 17, 23, 90], num_q_heads=hq, num_kv_heads=hkv, head_dim=D,
              pages_per_seq=32, sliding_window=window, max_num_seqs=96)
    out = to_np(run_hip(b, 0))
    assert_bf16_parity(out, run_strict(b), b.total_valid_tokens, f"decode-shaped {hq}/{hkv} D={D} W={window}")


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("window", [None, 48])
def test_bf16_first_visible_key_per_sequence(flags, window):
    """``RpaParams.kv_start`` (what ragged_decode_attention's ``sequence_start`` maps to) on every kind of work item:
    decode stream, few-row items and prefill tiles, with starts inside, at the edge of and past the visible range."""
    b = small([200, 1, 70, 130, 3, 1, 40], [200, 300, 100, 400, 90, 64, 40], pages_per_seq=32, sliding_window=window)
    starts = np.array([37, 250, 0, 399, 88, 64, 16], np.int32)   # 64 of 64: nothing visible for that sequence
    aux = torch.as_tensor(starts, device=DEV)
    out = RaggedPageAttention().run(*b.args(), softmax_scale=b.softmax_scale, sliding_window=b.sliding_window,
                                    cfg=RaggedPageAttentionConfig(), _flags=flags, _kv_start=aux)
    torch.cuda.synchronize()
    from oracle import rpa_oracle
    from tests.helpers import oracle_args

    ref = rpa_oracle.rpa_exact(*oracle_args(b), softmax_scale=b.softmax_scale, sliding_window=b.sliding_window,
                               kv_start=starts)
    assert_bf16_parity(to_np(out), ref, b.total_valid_tokens, f"kv_start W={window}")


@pytest.mark.parametrize("n_seqs,max_seqs", [(1500, 1500), (3000, 4096), (1025, 16384)])
def test_bf16_batches_of_more_than_1024_sequences(n_seqs, max_seqs):
    """Above 1024 sequences the schedule arrays keep every 2nd / 4th / 16th sequence's start: decode sequences, a few
    prefill chunks and empty sequences spread over the batch must all be found."""
    from oracle import rpa_oracle_c
    from tests.helpers import oracle_args

    rng = np.random.default_rng(n_seqs)
    q_lens = np.ones(n_seqs, int)
    kv_lens = rng.integers(1, 200, size=n_seqs)
    for s in rng.choice(n_seqs, size=12, replace=False):
        q_lens[s] = int(rng.integers(20, 90))
        kv_lens[s] = q_lens[s] + int(rng.integers(0, 100))
    for s in rng.choice(n_seqs, size=40, replace=False):
        q_lens[s] = 0
    b = small(q_lens, kv_lens, max_num_seqs=max_seqs, pages_per_seq=13)
    out = to_np(run_hip(b))
    ref = rpa_oracle_c.rpa_strict_c(*oracle_args(b), softmax_scale=b.softmax_scale)
    assert_bf16_parity(out, ref, b.total_valid_tokens, f"{n_seqs} sequences")
    assert not out[b.total_valid_tokens:].any()


@pytest.mark.parametrize("flags", PATHS)
def test_bf16_ragged_edge_cases(flags):
    """Empty sequences, kv_len not a page multiple, padding entries, garbage beyond the pages in use."""
    q_lens = [0, 1, 7, 0, 64, 1, 3, 130]
    kv_lens = [5, 1, 7, 16, 100, 241, 19, 131]
    b = small(q_lens, kv_lens, max_num_seqs=11)
    bt = b.block_tables.clone()
    for s, kl in enumerate(kv_lens):
        bt[s, -(-kl // 16):] = -1 if s % 2 else 2**30
    bt[len(q_lens):] = -5
    ref_b = Batch(**{**b.__dict__})
    b.block_tables = bt
    out = to_np(run_hip(b, flags))
    assert_bf16_parity(out, run_strict(ref_b), b.total_valid_tokens, "edge cases")
    assert not out[b.total_valid_tokens:].any()


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("window,cap", [(16, None), (100, None), (None, 30.0), (33, 5.0)])
def test_bf16_window_and_cap(flags, window, cap):
    b = small([4, 1, 1, 50], [200, 255, 40, 50], sliding_window=window, logits_soft_cap=cap)
    rows = b.total_valid_tokens
    strict = run_strict(b)
    assert np.isfinite(strict[:rows]).all()  # pages_per_seq < 64: one KV block, no NaN defect
    assert_bf16_parity(to_np(run_hip(b, flags)), strict, rows, f"window {window} cap {cap}")


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("shape", ["per_q", "per_kv", "shared"])
def test_bf16_sinks(flags, shape):
    b = small([4, 1, 1, 20], [200, 255, 1, 20])
    rng = np.random.default_rng(3)
    aux = {"per_q": rng.standard_normal((8, 2)), "per_kv": rng.standard_normal((2, 3)),
           "shared": rng.standard_normal(2)}[shape].astype(np.float32)
    # float32 sinks (what the ABI takes): the reference's epilogue is float32 with one final cast
    out32 = to_np(run_hip(b, flags, softmax_aux=torch.from_numpy(aux).to(DEV)))
    assert_bf16_parity(out32, run_strict(b, softmax_aux=aux, aux_dtype="float32"), b.total_valid_tokens,
                       f"float32 sinks {shape}")
    # sinks in the queries' bf16: the reference rounds every op of the epilogue to bf16
    aux_bf = torch.from_numpy(aux).to(torch.bfloat16)
    out = to_np(run_hip(b, flags, softmax_aux=aux_bf.to(DEV)))
    ref = run_strict(b, softmax_aux=aux_bf.float().numpy(), aux_dtype="bfloat16")
    assert_bf16_parity(out, ref, b.total_valid_tokens, f"sinks {shape}")
    base = to_np(run_hip(b, flags))
    assert np.abs(base - out)[: b.total_valid_tokens].max() > 1e-3  # sinks change the result


@pytest.mark.parametrize("seed", list(range(24)) + list(range(1000, 1120)))
def test_bf16_random_batches(seed):
    """Seeded random shapes on the MFMA path and on the scalar path: the parity bound against the op-by-op restatement
    on every row where that is finite (rows it turns NaN -- its first-KV-block defect under a window -- are left to
    the second check), and a bound of 4e-2 / 2e-3 against the float64 evaluation on every row (bf16 logits alone put
    up to 2.5e-2 between the restatement and float64 here).  Every path is held to the bound as it stands, the plain
    and the pipelined prefill tiles included; no element is excused by its distance from float64."""
    b, what = random_rpa_batch(seed, DEV)
    rows = b.total_valid_tokens
    strict, exact = run_strict(b)[:rows], run_exact(b)[:rows]
    finite = np.isfinite(strict).all(axis=(1, 2))
    for flags in (0, _native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES, _native.RPA_FLAG_PIPE_TILES,
                  _native.RPA_FLAG_FORCE_GENERIC):
        out = to_np(run_hip(b, flags))
        assert np.isfinite(out[:rows]).all(), what
        if finite.any():
            assert_bf16_parity_stepwise(out[:rows][finite], strict[finite], f"{what} flags={flags}")
        mx, mean = err_stats(out, exact, rows)
        assert mx <= 4e-2 and mean <= 2e-3, f"{what} flags={flags}: vs float64 max-abs {mx:.4g} mean-abs {mean:.4g}"
        assert not out[rows:].any()


@pytest.mark.parametrize("seed", range(60000, 60048))
def test_bf16_random_serving_batches(seed):
    """Seeded random serving steps -- long chunks whose few tiles have their key ranges cut, with and without decode
    steps beside them; small decode batches (one workgroup per (sequence, kv head)); a few very long decode sequences
    (the stream cut by workgroup) -- on the library's own choice of kernel: against the float64 evaluation where that
    takes a second or two (4e-2 / 2e-3, as for the other random batches: bf16 logits alone put 2.5e-2 between the
    reference's arithmetic and float64), against the wave-level loop with a caller-named split (which cuts no tile
    and merges no parts in LDS) to the parity bound, the same bits on a second call, zeros past the batch."""
    b, aux, hint, what = random_serving_batch(seed, DEV)
    rows = b.total_valid_tokens
    cfg = RaggedPageAttentionConfig(num_queries_per_block=hint) if hint else None
    out = run_hip(b, softmax_aux=aux, cfg=cfg)
    assert torch.equal(run_hip(b, softmax_aux=aux, cfg=cfg), out), what
    assert not out[rows:].any(), what
    page, pps = b.kv_pages.shape[1], b.block_tables.shape[1]
    by_wave = run_hip(b, softmax_aux=aux, cfg=RaggedPageAttentionConfig(num_queries_per_block=16,
                                                                         num_kv_pages_per_block=min(pps, max(1, 256 // page))))
    assert_bf16_parity_stepwise(to_np(out)[:rows], to_np(by_wave)[:rows], what + " (against the wave-level loop)")
    if sum(int(q) * int(k) for q, k in zip(b.q_lens, b.kv_lens)) * b.queries.shape[1] * b.queries.shape[2] <= 6e9:
        mx, mean = err_stats(to_np(out), run_exact(b, softmax_aux=aux), rows)
        assert mx <= 4e-2 and mean <= 2e-3, f"{what}: vs float64 max-abs {mx:.4g} mean-abs {mean:.4g}"


@pytest.mark.parametrize("seed", [8028, 8038, 9067])
def test_head_dim_64_prefill_tiles_on_seeds_that_once_showed_fp32_logits(seed):
    """Seeds found by sweeping new ones while the head_dim-64 prefill tiles kept fp32 logits: a row that sees a handful of
    keys then landed three bf16 steps from the restatement (0.0234).  The tiles round their logits where the reference
    does now, and the plain bound holds on the forced tiles as on the library's own choice."""
    b, what = random_rpa_batch(seed, DEV, head_dims=(64,))
    rows = b.total_valid_tokens
    strict = run_strict(b)[:rows]
    finite = np.isfinite(strict).all(axis=(1, 2))
    for flags in (_native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES, 0):
        out = to_np(run_hip(b, flags))
        assert_bf16_parity_stepwise(out[:rows][finite], strict[finite], f"{what} flags={flags}")


@pytest.mark.parametrize("seed", range(3000, 3040))
def test_bf16_random_batches_head_dims_between_the_instantiated_ones(seed):
    """head_dim 80, 96, 112 run on the 128-wide MFMA kernel and 144, 160, 192, 224 on the 256-wide one (q padded with
    zeros, the lanes past a row's last 16-byte piece fetching a piece that exists, output elements past head_dim not
    stored): same bounds as the other random batches, on the wave-level loop, the plain prefill tiles and the scalar
    kernel, and nothing written outside the rows of `out`."""
    b, what = random_rpa_batch(seed, DEV, head_dims=(80, 96, 112, 144, 160, 192, 224))
    rows = b.total_valid_tokens
    strict, exact = run_strict(b)[:rows], run_exact(b)[:rows]
    finite = np.isfinite(strict).all(axis=(1, 2))
    for flags in (0, _native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES, _native.RPA_FLAG_PIPE_TILES,
                  _native.RPA_FLAG_FORCE_GENERIC):
        out = to_np(run_hip(b, flags))
        assert np.isfinite(out[:rows]).all(), what
        if finite.any():
            assert_bf16_parity_stepwise(out[:rows][finite], strict[finite], f"{what} flags={flags}")
        mx, mean = err_stats(out, exact, rows)
        assert mx <= 4e-2 and mean <= 2e-3, f"{what} flags={flags}: vs float64 max-abs {mx:.4g} mean-abs {mean:.4g}"
        assert not out[rows:].any()


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("D", [16, 128])
def test_cap_that_bf16_does_not_hold_is_rounded_before_use(flags, D):
    """logits_soft_cap = 23.7 acts as 23.75 in the bf16 program (closed form in tests.helpers.two_key_cap_batch; with
    23.7 unrounded the result would be 0.6796875, nine bf16 steps away).  head_dim 16 runs on the scalar kernel."""
    b, want = two_key_cap_batch(DEV, head_dim=D)
    out = to_np(run_hip(b, flags))[0, 0]
    assert np.abs(out - want).max() <= 2.0 ** -8, out[:4]


@pytest.mark.parametrize("flags", PATHS)
def test_malformed_device_metadata_stays_in_bounds(flags):
    """A key count beyond what the block-table row can address, a negative one, and row offsets beyond the query
    buffer are clipped on the device (the reference's XLA program clamps every dynamic index; its Pallas path rejects
    such input, _pallas_impl_fwd.py:124-174): the rows of the well-formed sequences are bitwise what they are
    without the damage, nothing outside `out` is written, and the damaged sequences' rows are finite."""
    q_lens, kv_lens = [4, 1, 1, 50, 1, 3], [200, 255, 40, 50, 100, 64]
    b = small(q_lens, kv_lens, max_num_seqs=8)
    T, Hq, D = b.queries.shape
    base = run_hip(b, flags)
    # every buffer the damaged lengths could run past is a window into a larger allocation
    q_big = torch.zeros((T + 4096, Hq, D), dtype=b.queries.dtype, device=DEV)
    q_big[:T] = b.queries
    out_big = torch.full((T + 8192, Hq, D), 123.0, dtype=b.queries.dtype, device=DEV)
    bt_big = torch.zeros((8 + 64, b.block_tables.shape[1]), dtype=torch.int32, device=DEV)
    bt_big[:8] = b.block_tables
    bad = Batch(**{**b.__dict__})
    bad.queries, bad.block_tables = q_big[:T], bt_big[:8]
    bad.context_lens = b.context_lens.clone()
    bad.context_lens[1] = 100000        # 16 pages of 16 tokens can address 256 keys
    bad.context_lens[2] = -7            # no keys: zeros
    bad.query_start_loc = b.query_start_loc.clone()
    bad.query_start_loc[6:] = T + 1000  # the last sequence's rows run past the buffer: clipped at T
    out = RaggedPageAttention().run(*bad.args(), softmax_scale=b.softmax_scale, cfg=RaggedPageAttentionConfig(),
                                    _flags=flags, _out=out_big[4096:4096 + T])
    torch.cuda.synchronize()
    assert bool((out_big[:4096] == 123.0).all()) and bool((out_big[4096 + T:] == 123.0).all()), "wrote outside out"
    cu = np.concatenate([[0], np.cumsum(q_lens)])
    for s in (0, 3, 4):
        assert torch.equal(out[cu[s]:cu[s + 1]], base[cu[s]:cu[s + 1]]), f"well-formed sequence {s} changed"
    assert torch.isfinite(out.float()).all()
    assert not out[cu[2]:cu[3]].any(), "a sequence without keys yields zeros"
    # sequence 1 attends to the 256 keys its pages hold (one more than before)
    fixed = Batch(**{**b.__dict__})
    fixed.context_lens = b.context_lens.clone()
    fixed.context_lens[1] = 256
    fixed.kv_lens = np.array(kv_lens)
    fixed.kv_lens[1] = 256
    assert_bf16_parity(to_np(out[cu[1]:cu[2]]), run_strict(fixed)[cu[1]:cu[2]], 1, "clipped key count")
    # the last sequence keeps the rows that exist: with kv_len 64 and a (damaged) q_len beyond it, row r sits at
    # position 64 - q_len + r of the clipped chunk
    assert out.shape[0] == T


# ----------------------------------------------------------------------------- invariants on the device result


@pytest.mark.parametrize("flags", PATHS)
def test_window_covering_everything_equals_no_window(flags):
    b = small([4, 1, 1, 50], [200, 255, 40, 50])
    base = run_hip(b, flags)
    b.sliding_window = 256
    assert torch.equal(run_hip(b, flags), base)
    b.logits_soft_cap = 1e6  # cap far above any logit: tanh is linear there
    d = (run_hip(b, flags).float() - base.float()).abs().max().item()
    assert d < 0.1, d  # bound of the reference's own property test (test_ragged_page_attention.py:437-461)


@pytest.mark.parametrize("flags", PATHS)
def test_page_permutation_invariance_is_bitwise(flags):
    b = make_workload("mixed_prefill_decode", device=DEV, scale=0.08)
    base = run_hip(b, flags)
    P = b.kv_pages.shape[0]
    perm = torch.randperm(P, generator=torch.Generator().manual_seed(9)).to(DEV)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(P, device=DEV)
    b2 = Batch(**{**b.__dict__})
    b2.kv_pages = b.kv_pages[perm].contiguous()
    b2.block_tables = inv[b.block_tables.long()].to(torch.int32)
    assert torch.equal(run_hip(b2, flags), base)


@pytest.mark.parametrize("flags", PATHS)
def test_rows_do_not_depend_on_batch_composition(flags):
    b = small([4, 1, 1, 50, 1], [200, 255, 40, 50, 90], max_num_seqs=7)
    full = run_hip(b, flags)
    cu = b.query_start_loc.cpu().numpy()
    for s in (1, 3, 4):
        sub = compact_for_host(b, [s])
        sub_dev = Batch(**{**sub.__dict__})
        for f in ("queries", "kv_pages", "context_lens", "block_tables", "query_start_loc", "num_seqs"):
            setattr(sub_dev, f, getattr(sub, f).to(DEV))
        alone = run_hip(sub_dev, flags)
        n = int(b.q_lens[s])
        # the same math; a different share of the decode stream may split the keys elsewhere, which can flip the
        # last place of a bf16 result
        d = (alone[:n].float() - full[cu[s]:cu[s] + n].float()).abs().max().item()
        assert d <= 2.0 ** -7 * max(1.0, full[cu[s]:cu[s] + n].float().abs().max().item()), (s, d)


def test_repeated_calls_are_deterministic():
    b = make_workload("decode_llama3_8b", device=DEV, scale=0.1)
    a = run_hip(b)
    for _ in range(3):
        assert torch.equal(run_hip(b), a)


def test_module_function_is_the_same_path():
    b = small([4, 1], [200, 255])
    a = ragged_page_attention(*b.args(), softmax_scale=b.softmax_scale)
    torch.cuda.synchronize()
    assert torch.equal(a, run_hip(b))
    c = ragged_page_attention(b.queries, b.kv_pages, b.context_lens, b.block_tables, b.query_start_loc, 2)
    torch.cuda.synchronize()
    assert torch.equal(a, c)  # num_seqs may be a plain int; scale defaults to head_dim ** -0.5


def test_non_default_stream():
    b = small([4, 1], [200, 255])
    base = run_hip(b)
    st = torch.cuda.Stream()
    with torch.cuda.stream(st):
        out = ragged_page_attention(*b.args(), softmax_scale=b.softmax_scale)
    st.synchronize()
    assert torch.equal(out, base)


def test_concurrent_streams_do_not_share_a_workspace():
    """Two streams run split sequences (partial results and tickets in the workspace) at the same time; each stream has
    a workspace of its own, so every result equals the one computed alone, bit for bit."""
    batches = [make_workload("decode_long_context", device=DEV, scale=0.05), make_workload("mixed_prefill_decode", device=DEV, scale=0.1)]
    alone = [run_hip(b) for b in batches]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    outs = [[], []]
    for _ in range(8):
        for k in range(2):
            with torch.cuda.stream(streams[k]):
                outs[k].append(ragged_page_attention(*batches[k].args(), **batches[k].kwargs()))
    torch.cuda.synchronize()
    for k in range(2):
        for o in outs[k]:
            assert torch.equal(o, alone[k])


def test_host_threads_launch_at_the_same_time_on_streams_of_their_own():
    """The C entry points are re-entrant (error text per thread, tuning knobs and kernel attributes set once under a
    guard) and ctypes drops the interpreter lock around them, so two host threads really launch at once; every result
    equals the one computed alone, bit for bit, and an error raised in one thread names that thread's mistake."""
    import threading

    batches = [make_workload("decode_long_context", device=DEV, scale=0.05), make_workload("mixed_prefill_decode", device=DEV, scale=0.1)]
    alone = [run_hip(b) for b in batches]
    torch.cuda.synchronize()
    failures = []

    def work(k):
        try:
            torch.cuda.set_device(0)
            st = torch.cuda.Stream()
            with torch.cuda.stream(st):
                for rep in range(12):
                    out = ragged_page_attention(*batches[k].args(), **batches[k].kwargs())
                    if rep % 4 == 3:
                        st.synchronize()
                        if not torch.equal(out, alone[k]):
                            failures.append((k, rep, "result differs"))
                bad = batches[k]
                try:  # a rejected call in this thread: the message is this thread's
                    ragged_page_attention(bad.queries, bad.kv_pages, bad.context_lens, bad.block_tables, bad.query_start_loc,
                                          bad.num_seqs, softmax_scale=float("nan") if k == 0 else 1.0,
                                          logits_soft_cap=None if k == 0 else float("nan"))
                    failures.append((k, "no error"))
                except (ValueError, RuntimeError) as e:
                    if ("softmax_scale is NaN" if k == 0 else "logits_soft_cap is NaN") not in str(e):
                        failures.append((k, str(e)))
            st.synchronize()
        except Exception as e:  # noqa: BLE001
            failures.append((k, repr(e)))

    threads = [threading.Thread(target=work, args=(k,)) for k in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not failures, failures


def test_workspace_cache_is_bounded_over_many_streams():
    """Every (device, stream) gets its own workspace; past the bound the least recently used one is dropped, and a call on
    a stream whose workspace was dropped allocates (and clears) a new one."""
    import importlib

    m = importlib.import_module("ejkernel_amd.modules.operations.ragged_page_attention")
    b = small([1, 3, 1], [100, 90, 17])
    want = to_np(run_hip(b))
    streams = [torch.cuda.Stream() for _ in range(m._MAX_WORKSPACES + 4)]
    for st in streams + streams[:2]:
        with torch.cuda.stream(st):
            out = RaggedPageAttention().run(*b.args(), softmax_scale=b.softmax_scale, cfg=RaggedPageAttentionConfig())
        st.synchronize()
        assert np.array_equal(to_np(out), want)
        assert len(m._workspaces) <= m._MAX_WORKSPACES


def test_launch_recorded_in_a_hip_graph_replays_correctly():
    """The launch only enqueues (no allocation, no synchronisation, tickets and queue counters left at zero), so it can
    be captured; every replay on new input values must equal the eager result bit for bit."""
    b = make_workload("mixed_prefill_decode", device=DEV, scale=0.05)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            ragged_page_attention(*b.args(), **b.kwargs())
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out_g = ragged_page_attention(*b.args(), **b.kwargs())
    gen = torch.Generator(device=DEV).manual_seed(5)
    for rep in range(4):
        b.queries.copy_(torch.randn(b.queries.shape, generator=gen, device=DEV).to(b.queries.dtype))
        if rep == 2:  # other K/V values too
            b.kv_pages.mul_(-1)
        want = ragged_page_attention(*b.args(), **b.kwargs())
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out_g, want), rep


def test_bf16_call_on_the_scalar_kernel_warns_once_per_shape():
    """A bf16 call the MFMA kernels do not take (here: pages of 2 tokens) runs on the scalar kernel, exact and far
    slower: the Python layer says so the first time it sees the shape, and not again."""
    import warnings

    import importlib

    from ejkernel_amd.modules import ragged_page_attention

    m = importlib.import_module("ejkernel_amd.modules.operations.ragged_page_attention")
    b = small([3, 1], [9, 30], page_size=2, pages_per_seq=16, head_dim=128)
    m._warned_scalar.discard((128, 2, b.block_tables.shape[0]))
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        out = ragged_page_attention(*b.args(), **b.kwargs())
        ragged_page_attention(*b.args(), **b.kwargs())
    torch.cuda.synchronize()
    assert len([w for w in seen if "scalar kernel" in str(w.message)]) == 1
    assert_bf16_parity(to_np(out), run_strict(b), b.total_valid_tokens, "pages of 2 tokens")
    ok = small([3, 1], [9, 30], page_size=4, pages_per_seq=8, head_dim=128)
    with warnings.catch_warnings(record=True) as seen:
        warnings.simplefilter("always")
        ragged_page_attention(*ok.args(), **ok.kwargs())
    assert not [w for w in seen if "scalar kernel" in str(w.message)]
