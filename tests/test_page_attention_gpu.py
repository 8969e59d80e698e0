"""page_attention on the device (through ``rpa_page_attention_launch``) against its CPU oracle.

bf16 with an explicit scale: max-abs <= 2e-2 / mean-abs <= 2e-3 against the op-by-op restatement of the reference's
XLA program.  Default scale (the reference computes in float32 then): the same bound against the float32
restatement.  float32 inputs: <= 1e-5 against the float64 dense evaluation.  Each case on the MFMA path and on the
scalar path.
"""

import numpy as np
import pytest
import torch

from ejkernel_amd import _native
from ejkernel_amd.modules import PageAttentionConfig, page_attention
from ejkernel_amd.workloads import make_page_attention_batch, page_attention_subset, page_attention_workload
from oracle.page_attention_oracle import page_attention_exact, page_attention_strict
from tests.helpers import F32_MAX_ABS, assert_bf16_parity, assert_bf16_parity_stepwise, err_stats, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PATHS = [pytest.param(0, id="tiled"), pytest.param(_native.RPA_FLAG_FORCE_GENERIC, id="generic")]


def small(kv_lens, **kw):
    args = dict(num_q_heads=8, num_kv_heads=2, head_dim=128, block_size=16, max_blocks=20, seed=11, device=DEV)
    args.update(kw)
    return make_page_attention_batch(kv_lens, **args)


def np_args(b):
    return [to_np(t) for t in b.args()]


def run_hip(b, flags=0, **kw):
    out = page_attention(*b.args(), _flags=flags, **kw)
    torch.cuda.synchronize()
    return to_np(out)


KV = [1, 15, 16, 17, 100, 255, 256, 300, 64]


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("kw", [dict(), dict(num_q_heads=8, num_kv_heads=8), dict(num_q_heads=32, num_kv_heads=1),
                                dict(head_dim=256, num_q_heads=16, num_kv_heads=8), dict(block_size=4, max_blocks=80),
                                dict(block_size=64, max_blocks=5), dict(head_dim=64),
                                dict(num_q_heads=80, num_kv_heads=1)],
                         ids=["gqa4", "mha", "mqa32", "d256", "block4", "block64", "d64", "mqa80"])
def test_bf16_explicit_scale(kw, flags):
    b = small(KV, **kw)
    ref = page_attention_strict(*np_args(b), attn_scale=b.attn_scale)
    assert_bf16_parity(run_hip(b, flags, attn_scale=b.attn_scale), ref, len(KV), str(kw))


@pytest.mark.parametrize("flags", PATHS)
def test_bf16_default_scale_follows_the_float32_promotion(flags):
    b = small(KV)
    ref = page_attention_strict(*np_args(b), attn_scale=None)
    mx, mean = assert_bf16_parity(run_hip(b, flags), ref, len(KV), "default scale")
    assert mx <= 1e-2  # only the bf16 rounding of P and of the output (half an ulp of values up to 4) separates the two


@pytest.mark.parametrize("flags", PATHS)
def test_float32_against_float64(flags):
    b = small(KV, dtype=torch.float32)
    mx, _ = err_stats(run_hip(b, flags, attn_scale=0.07), page_attention_exact(*np_args(b), attn_scale=0.07), len(KV))
    assert mx <= F32_MAX_ABS, mx


@pytest.mark.parametrize("flags", PATHS)
def test_single_key_is_bit_exact_and_empty_context_gives_zeros(flags):
    b = small([1, 0, 1, 1])
    out = page_attention(*b.args(), attn_scale=0.1, _flags=flags)
    bt = b.block_tables.long()
    want = b.value_cache[bt[:, 0], :, 0, :].repeat_interleave(4, dim=1)
    for s in (0, 2, 3):
        assert torch.equal(out[s], want[s])
    assert not out[1].any()


@pytest.mark.parametrize("flags", PATHS)
def test_block_permutation_is_bitwise_invariant_and_tail_entries_are_ignored(flags):
    b = small(KV)
    out = page_attention(*b.args(), attn_scale=b.attn_scale, _flags=flags)
    nb = b.key_cache.shape[0]
    perm = torch.randperm(nb, generator=torch.Generator().manual_seed(3)).to(DEV)
    inv = torch.empty_like(perm)
    inv[perm] = torch.arange(nb, device=DEV)
    bt2 = inv[b.block_tables.long()].to(torch.int32)
    used = (torch.arange(bt2.shape[1], device=DEV)[None, :] * 16) < b.context_lens[:, None]
    bt2 = torch.where(used, bt2, torch.full_like(bt2, -1))  # garbage past the context
    out2 = page_attention(b.query, b.key_cache[perm], b.value_cache[perm], b.context_lens, bt2,
                          attn_scale=b.attn_scale, _flags=flags)
    assert torch.equal(out, out2)


def test_same_rows_as_ragged_page_attention_on_the_interleaved_layout():
    from ejkernel_amd.modules import ragged_page_attention

    b = small(KV)
    S = len(KV)
    k = b.key_cache.permute(0, 2, 1, 3)
    v = b.value_cache.permute(0, 2, 1, 3)
    pages = torch.stack([k, v], dim=3).reshape(k.shape[0], k.shape[1], -1, k.shape[3]).contiguous()
    out2 = ragged_page_attention(b.query, pages, b.context_lens, b.block_tables,
                                 torch.arange(S + 1, dtype=torch.int32, device=DEV),
                                 torch.tensor([S], dtype=torch.int32, device=DEV), softmax_scale=b.attn_scale)
    out = page_attention(*b.args(), attn_scale=b.attn_scale)
    assert torch.equal(out, out2[:S])   # same kernel, same arithmetic, another addressing


def test_arguments_the_reference_backend_rejects():
    b = small([5, 9])
    for kw in (dict(max_context_len=128), dict(num_splits=2), dict(pages_per_compute_block=4),
               dict(megacore_mode="kv_head"), dict(inline_seq_dim=False), dict(attn_logits_soft_cap=30.0)):
        with pytest.raises(NotImplementedError, match="not supported in XLA implementation"):
            page_attention(*b.args(), **kw)
    with pytest.raises(ValueError):
        page_attention(b.query, b.key_cache, b.value_cache[:, :1], b.context_lens, b.block_tables)
    with pytest.raises(ValueError):
        page_attention(*b.args(), cfg=PageAttentionConfig(platform="tpu"))


@pytest.mark.parametrize("name,n_sample", [("decode_small", 8), ("decode_llama3_8b", 12)])
def test_full_size_workload(name, n_sample):
    b = page_attention_workload(name, device=DEV)
    out = page_attention(*b.args(), attn_scale=b.attn_scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out, page_attention(*b.args(), attn_scale=b.attn_scale))   # reproducible bit for bit
    rng = np.random.default_rng(0)
    ids = sorted(int(s) for s in rng.permutation(len(b.kv_lens))[:n_sample])
    sub = page_attention_subset(b, ids)
    ref = page_attention_strict(*np_args(sub), attn_scale=b.attn_scale)
    assert_bf16_parity(to_np(out[sub.meta["rows"].to(DEV)]), ref, len(ids), name)


@pytest.mark.parametrize("seed", range(200, 228))
def test_bf16_random_batches(seed):
    """Seeded random shapes on both paths against the restatement of the reference program (explicit scale); from seed
    216 on at head dims between the instantiated ones."""
    rng = np.random.default_rng(seed)
    hq, hkv = [(8, 2), (4, 4), (16, 2), (32, 8), (8, 1), (40, 1), (12, 4)][rng.integers(7)]
    D = int(rng.choice([64, 128, 256]))
    if seed >= 216:
        D = int(rng.choice([80, 96, 112, 160, 192]))
    bs = int(rng.choice([4, 8, 16, 32, 64]))
    n = int(rng.integers(1, 12))
    kv = [int(rng.integers(1, 500)) for _ in range(n)]       # context_len 0 is garbage in the reference: not drawn
    mb = -(-max(kv) // bs) + int(rng.integers(0, 3))
    b = make_page_attention_batch(kv, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, block_size=bs, max_blocks=mb,
                                  seed=seed, device=DEV)
    scale = float(rng.choice([D ** -0.5, 0.05, 0.2]))
    ref = page_attention_strict(*np_args(b), attn_scale=scale)
    for flags in (0, _native.RPA_FLAG_FORCE_GENERIC):
        assert_bf16_parity_stepwise(run_hip(b, flags, attn_scale=scale), ref,
                                    f"seed {seed}: {hq}/{hkv} D={D} block={bs} kv={kv} scale={scale:.3g} flags={flags}")
