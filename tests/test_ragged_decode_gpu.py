"""ragged_decode_attention on the device (through ``rpa_ragged_decode_launch``) against its CPU oracle.

Where the reference's XLA program is attention -- sequences inside one KV block whose first block has a visible
key -- bf16 outputs are within max-abs 2e-2 / mean-abs 2e-3 of its op-by-op restatement.  Everywhere (several
blocks, starts past the first block, windows: the program is off or NaN there) they are held to the same bound
against the float64 dense evaluation.  float32 inputs: <= 1e-5 against float64.
"""

import numpy as np
import pytest
import torch

from ejkernel_amd import _native
from ejkernel_amd.modules import RaggedDecodeAttentionConfig, ragged_decode_attention
from ejkernel_amd.workloads import make_ragged_decode_batch, ragged_decode_workload
from oracle.ragged_decode_oracle import ragged_decode_exact, ragged_decode_strict
from tests.helpers import F32_MAX_ABS, assert_bf16_parity, assert_bf16_parity_stepwise, err_stats, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PATHS = [pytest.param(0, id="tiled"), pytest.param(_native.RPA_FLAG_FORCE_GENERIC, id="generic")]


def small(starts, ends, **kw):
    args = dict(seq_len=320, num_q_heads=8, num_kv_heads=2, head_dim=128, seed=13, device=DEV)
    args.update(kw)
    return make_ragged_decode_batch(starts, ends, **args)


def np_args(b):
    return [to_np(t) for t in b.args()]


def run_hip(b, flags=0, **kw):
    out = ragged_decode_attention(*b.args(), softmax_scale=b.softmax_scale, _flags=flags, **kw)
    torch.cuda.synchronize()
    return to_np(out)


ENDS = [1, 15, 16, 17, 100, 255, 256, 300, 64]


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("kw", [dict(), dict(num_q_heads=8, num_kv_heads=8), dict(num_q_heads=32, num_kv_heads=1),
                                dict(head_dim=256, num_q_heads=16, num_kv_heads=8), dict(head_dim=64), dict(seq_len=301),
                                dict(num_q_heads=80, num_kv_heads=1)],
                         ids=["gqa4", "mha", "mqa32", "d256", "d64", "odd_seq_len", "mqa80"])
def test_bf16_against_the_reference_program_on_one_block(kw, flags):
    b = small(np.zeros(len(ENDS), int), ENDS, **kw)
    ref = ragged_decode_strict(*np_args(b), softmax_scale=b.softmax_scale, block_size=512)
    assert_bf16_parity(run_hip(b, flags), ref, len(ENDS), str(kw))


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("window,cap", [(None, None), ((40, 0), None), ((7, 3), None), (None, 20.0), ((100, 0), 5.0)])
def test_bf16_starts_windows_and_caps_against_float64(flags, window, cap):
    starts = [0, 3, 16, 0, 99, 200, 31, 290, 64]       # the last one is empty (start == end)
    b = small(starts, ENDS[:-1] + [64])
    b.sequence_start[:] = torch.tensor(np.minimum(starts, b.ends), dtype=torch.int32)
    ref = ragged_decode_exact(*np_args(b), softmax_scale=b.softmax_scale, sliding_window=window, logits_soft_cap=cap)
    out = run_hip(b, flags, sliding_window=window, logits_soft_cap=cap)
    assert_bf16_parity(out, ref, len(ENDS), f"window {window} cap {cap}")
    assert not out[8].any()                           # nothing visible: zeros


@pytest.mark.parametrize("flags", PATHS)
def test_sequence_end_beyond_the_cache_is_clipped(flags):
    """sequence_end > seq_len must not read the next sequence's keys (or past the buffers for the last sequence): the
    reference masks with arange(seq_len) (_xla_impl_fwd.py:50-55), so such an end acts as seq_len; the device clips it.
    Without a window the two agree on every row."""
    ends = [300, 64, 320, 17, 200]
    b = small([0, 5, 100, 0, 7], ends)
    want = run_hip(b, flags)
    big_k = torch.zeros((len(ends) + 2, *b.key.shape[1:]), dtype=b.key.dtype, device=DEV)
    big_v = torch.zeros_like(big_k)
    big_k[:len(ends)], big_v[:len(ends)] = b.key, b.value
    big_k[len(ends):] = float("nan")  # what a read past the last sequence would see
    big_v[len(ends):] = float("nan")
    end_bad = b.sequence_end.clone()
    end_bad[2] = 320 + 5000           # already the whole cache: nothing changes
    end_bad[4] = 2 ** 30              # the last sequence: acts as seq_len = 320
    out = ragged_decode_attention(b.query, big_k[:len(ends)], big_v[:len(ends)], b.sequence_start, end_bad,
                                  softmax_scale=b.softmax_scale, _flags=flags)
    torch.cuda.synchronize()
    out = to_np(out)
    assert np.isfinite(out).all()
    assert np.array_equal(out[:4], want[:4])
    ref = ragged_decode_exact(to_np(b.query), to_np(b.key), to_np(b.value), to_np(b.sequence_start),
                              np.array([300, 64, 320, 17, 320], np.int32), softmax_scale=b.softmax_scale)
    assert_bf16_parity(out, ref, len(ends), "clipped sequence_end")


@pytest.mark.parametrize("flags", PATHS)
def test_float32_against_float64(flags):
    b = small([0, 5, 100, 0], [300, 64, 101, 17], dtype=torch.float32)
    ref = ragged_decode_exact(*np_args(b), softmax_scale=b.softmax_scale, sliding_window=(150, 0))
    mx, _ = err_stats(run_hip(b, flags, sliding_window=(150, 0)), ref, 4)
    assert mx <= F32_MAX_ABS, mx


@pytest.mark.parametrize("flags", PATHS)
def test_single_visible_key_is_bit_exact(flags):
    b = small([9, 0, 255], [10, 1, 256])
    out = ragged_decode_attention(*b.args(), softmax_scale=0.1, _flags=flags)
    for s, pos in enumerate([9, 0, 255]):
        assert torch.equal(out[s], b.value[s, pos].repeat_interleave(4, dim=0))
    out = ragged_decode_attention(*small([0, 0], [200, 33]).args(), sliding_window=(0, 0), _flags=flags)
    b2 = small([0, 0], [200, 33])
    assert torch.equal(out[0], b2.value[0, 199].repeat_interleave(4, dim=0))
    assert torch.equal(out[1], b2.value[1, 32].repeat_interleave(4, dim=0))


def test_query_with_a_singleton_axis_and_rejected_arguments():
    b = small([0, 4], [50, 20])
    out = ragged_decode_attention(*b.args())
    out4 = ragged_decode_attention(b.query[:, None], *b.args()[1:])
    assert out4.shape == (2, 1, 8, 128) and torch.equal(out4[:, 0], out)
    with pytest.raises(ValueError, match="broadcast"):   # [num_kv_heads, num_sinks] with 4 query heads per kv head
        ragged_decode_attention(*b.args(), torch.zeros(2, 4, device=DEV))
    with pytest.raises(ValueError, match="at most"):
        ragged_decode_attention(*b.args(), torch.zeros(65, device=DEV))
    assert torch.equal(ragged_decode_attention(*b.args(), torch.zeros(0, device=DEV)), out)
    with pytest.raises(ValueError):
        ragged_decode_attention(*b.args(), sliding_window=(-1, 0))
    with pytest.raises(ValueError):
        ragged_decode_attention(*b.args()[:4], b.sequence_end.long())
    with pytest.raises(ValueError):
        ragged_decode_attention(*b.args(), cfg=RaggedDecodeAttentionConfig(platform="tpu"))
    with pytest.raises(NotImplementedError):
        ragged_decode_attention(*b.args(), mesh=object())


# ---- attention sinks (softmax_aux): keys [start, start + num_sinks) always visible, bias on absolute t < num_sinks

SINK_STARTS = [0, 2, 16, 0, 99, 200, 31, 290, 64, 318]
SINK_ENDS = [1, 15, 16, 300, 100, 255, 256, 300, 64, 320]   # 2: empty, 8: empty, 9: sink range cut by seq_len


def sink_batch(**kw):
    return small(SINK_STARTS, SINK_ENDS, **kw)


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("window,cap", [(None, None), ((40, 0), None), ((0, 0), None), ((100, 0), 5.0)])
@pytest.mark.parametrize("aux_kind", ["vector", "per_group_head"])
def test_bf16_sinks_against_float64(flags, window, cap, aux_kind):
    b = sink_batch()
    g = torch.Generator().manual_seed(3)
    aux = (torch.randn(5, generator=g) if aux_kind == "vector" else torch.randn(4, 5, generator=g)) * 2.0
    ref = ragged_decode_exact(*np_args(b), softmax_scale=b.softmax_scale, sliding_window=window, logits_soft_cap=cap,
                              softmax_aux=aux.numpy())
    out = to_np(ragged_decode_attention(*b.args(), aux.to(DEV), softmax_scale=b.softmax_scale, sliding_window=window,
                                        logits_soft_cap=cap, _flags=flags))
    assert_bf16_parity(out, ref, len(SINK_ENDS), f"sinks {aux_kind} window {window} cap {cap}")
    assert out[2].any() and out[8].any()               # an empty sequence still attends to its sink range


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("kw", [dict(num_q_heads=8, num_kv_heads=8), dict(num_q_heads=32, num_kv_heads=1),
                                dict(head_dim=256, num_q_heads=16, num_kv_heads=8), dict(head_dim=64)],
                         ids=["mha", "mqa32", "d256", "d64"])
def test_bf16_sinks_against_the_reference_program_on_one_block(kw, flags):
    b = small(np.zeros(len(ENDS), int), ENDS, **kw)
    aux = torch.tensor([1.5, -0.5, 3.0, 0.25])
    ref = ragged_decode_strict(*np_args(b), softmax_scale=b.softmax_scale, block_size=512, softmax_aux=aux.numpy())
    out = to_np(ragged_decode_attention(*b.args(), aux.to(DEV), softmax_scale=b.softmax_scale, _flags=flags))
    assert_bf16_parity(out, ref, len(ENDS), f"sinks {kw}")


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("ns,kw", [(9, dict()), (24, dict(head_dim=64)), (64, dict(head_dim=256, num_q_heads=16, num_kv_heads=8)),
                                   (33, dict(num_q_heads=32, num_kv_heads=2)), (11, dict(head_dim=96)), (8, dict(head_dim=80)),
                                   (12, dict(head_dim=112)), (10, dict(head_dim=144, num_q_heads=16, num_kv_heads=8)),
                                   (9, dict(head_dim=224))],
                         ids=["9", "24-d64", "64-d256", "33-g16", "11-d96", "8-d80", "12-d112", "10-d144", "9-d224"])
def test_bf16_many_sinks_against_float64(flags, ns, kw):
    """More sink keys than the attention kernel stages per wavefront (8): the rest is read key by key; per-head biases,
    a sink range cut by seq_len (sequence 9) and by nothing else (sequences 2 and 8 are empty but for their sinks)."""
    b = sink_batch(**kw)
    G = b.query.shape[1] // b.key.shape[2]
    aux = torch.randn(G, ns, generator=torch.Generator().manual_seed(ns)) * 2.0
    ref = ragged_decode_exact(*np_args(b), softmax_scale=b.softmax_scale, sliding_window=(50, 0), softmax_aux=aux.numpy())
    out = to_np(ragged_decode_attention(*b.args(), aux.to(DEV), softmax_scale=b.softmax_scale, sliding_window=(50, 0),
                                        _flags=flags))
    assert_bf16_parity(out, ref, len(SINK_ENDS), f"{ns} sinks {kw}")


@pytest.mark.parametrize("flags", PATHS)
@pytest.mark.parametrize("hq,hkv,ns", [(40, 1, 5), (24, 2, 3), (40, 1, 11), (64, 2, 2)])
def test_bf16_per_head_sinks_with_more_than_16_query_heads_per_kv_head(flags, hq, hkv, ns):
    """More than 16 query heads per kv head: a decode token's rows take several 16-row tiles, and each tile needs the
    bias rows of its own query heads (rows 16 and up once read those of rows 0..15: found by a sweep of new seeds)."""
    b = sink_batch(num_q_heads=hq, num_kv_heads=hkv)
    aux = torch.randn(hq // hkv, ns, generator=torch.Generator().manual_seed(hq + ns)) * 2.0
    ref = ragged_decode_exact(*np_args(b), softmax_scale=b.softmax_scale, sliding_window=(60, 0), softmax_aux=aux.numpy())
    out = to_np(ragged_decode_attention(*b.args(), aux.to(DEV), softmax_scale=b.softmax_scale, sliding_window=(60, 0),
                                        _flags=flags))
    assert_bf16_parity(out, ref, len(SINK_ENDS), f"{hq}/{hkv} with {ns} sinks per head")


@pytest.mark.parametrize("flags", PATHS)
def test_float32_sinks_against_float64(flags):
    b = sink_batch(dtype=torch.float32)
    aux = torch.tensor([[0.5, -1.0, 2.0]])
    ref = ragged_decode_exact(*np_args(b), softmax_scale=b.softmax_scale, sliding_window=(30, 0), softmax_aux=aux.numpy())
    out = to_np(ragged_decode_attention(*b.args(), aux.to(DEV), softmax_scale=b.softmax_scale, sliding_window=(30, 0),
                                        _flags=flags))
    mx, _ = err_stats(out, ref, len(SINK_ENDS))
    assert mx <= F32_MAX_ABS, mx


@pytest.mark.parametrize("flags", PATHS)
def test_sink_closed_forms_on_the_device(flags):
    # q = 0 and a window that keeps the query position only: weights e^{a_t} on the sink range, 1 on the query position
    b = small([0, 5], [200, 200], dtype=torch.float32)
    b.query.zero_()
    aux = torch.tensor([0.75, -0.5])
    out = ragged_decode_attention(*b.args(), aux.to(DEV), sliding_window=(0, 0), _flags=flags).double()
    v = b.value.double()
    w0, w1 = float(np.exp(0.75)), float(np.exp(-0.5))
    want0 = (w0 * v[0, 0] + w1 * v[0, 1] + v[0, 199]) / (w0 + w1 + 1.0)
    want1 = (v[1, 5] + v[1, 6] + v[1, 199]) / 3.0     # the sink range {5, 6} lies past the biased positions
    assert (out[0] - want0.repeat_interleave(4, dim=0)).abs().max() <= 1e-6
    assert (out[1] - want1.repeat_interleave(4, dim=0)).abs().max() <= 1e-6
    # biases of zero on keys that are visible anyway change nothing at all
    b = small([0, 3], [300, 77])
    plain = ragged_decode_attention(*b.args(), _flags=flags)
    zeros = ragged_decode_attention(*b.args(), torch.zeros(4, device=DEV), _flags=flags)
    assert (plain.float() - zeros.float()).abs().max() <= 8e-3   # same keys, split at another point: one bf16 ulp


def test_sinks_full_size_workload():
    b = ragged_decode_workload("decode_llama3_8b", device=DEV)
    aux = torch.linspace(-1.0, 2.0, 4)
    out = ragged_decode_attention(*b.args(), aux.to(DEV), softmax_scale=b.softmax_scale, sliding_window=(1023, 0))
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out, ragged_decode_attention(*b.args(), aux.to(DEV), softmax_scale=b.softmax_scale,
                                                    sliding_window=(1023, 0)))
    ids = torch.tensor(sorted(int(s) for s in np.random.default_rng(1).permutation(len(b.ends))[:8]))
    sub = [to_np(t[ids.to(DEV)]) for t in b.args()]
    ref = ragged_decode_exact(*sub, softmax_scale=b.softmax_scale, sliding_window=(1023, 0), softmax_aux=aux.numpy())
    assert_bf16_parity(to_np(out[ids.to(DEV)]), ref, len(ids), "decode_llama3_8b with sinks")


@pytest.mark.parametrize("name,n_sample", [("decode_small", 8), ("decode_llama3_8b", 10)])
def test_full_size_workload(name, n_sample):
    b = ragged_decode_workload(name, device=DEV)
    out = ragged_decode_attention(*b.args(), softmax_scale=b.softmax_scale)
    torch.cuda.synchronize()
    assert torch.isfinite(out.float()).all()
    assert torch.equal(out, ragged_decode_attention(*b.args(), softmax_scale=b.softmax_scale))
    rng = np.random.default_rng(0)
    ids = torch.tensor(sorted(int(s) for s in rng.permutation(len(b.ends))[:n_sample]))
    sub = [to_np(t[ids.to(DEV)]) for t in b.args()]
    ref = ragged_decode_exact(*sub, softmax_scale=b.softmax_scale)
    assert_bf16_parity(to_np(out[ids.to(DEV)]), ref, len(ids), name)


@pytest.mark.parametrize("seed", [*range(300, 340), 11103, 11155, 20206, 20234])
def test_bf16_random_batches(seed):
    """Seeded random shapes, starts, ends, windows, caps and sinks on both paths: within the parity bound of the
    reference program's restatement with one KV block per sequence on the rows it keeps finite, and within 4e-2 / 2e-3 of
    the float64 evaluation everywhere."""
    rng = np.random.default_rng(seed)
    hq, hkv = [(8, 2), (4, 4), (16, 2), (32, 8), (8, 1), (40, 1), (12, 4)][rng.integers(7)]
    D = int(rng.choice([64, 128, 256]))
    if seed >= 324:  # head dims between the instantiated ones (rows whose 16-byte pieces are no power of two in number)
        D = int(rng.choice([80, 96, 112, 160, 192]))
    S = int(rng.integers(1, 400))
    n = int(rng.integers(1, 10))
    ends = rng.integers(0, S + 1, size=n)
    starts = np.minimum(rng.integers(0, S + 1, size=n) * (rng.random(n) < 0.5), ends + rng.integers(0, 3, size=n))
    starts = np.minimum(starts, S)
    window = None if rng.random() < 0.5 else (int(rng.integers(0, 120)), int(rng.integers(0, 5)))
    cap = None if rng.random() < 0.6 else float(rng.choice([5.0, 20.0, 50.0]))
    G = hq // hkv
    aux = None
    if rng.random() < 0.6:
        ns = int(rng.integers(1, 7))
        aux = (rng.standard_normal((int(rng.choice([1, G])), ns)) * 2).astype(np.float32)
        if rng.random() < 0.3:
            aux = aux[0]
    b = make_ragged_decode_batch(starts, ends, seq_len=S, num_q_heads=hq, num_kv_heads=hkv, head_dim=D, seed=seed,
                                 device=DEV)
    what = f"seed {seed}: {hq}/{hkv} D={D} S={S} starts={list(starts)} ends={list(ends)} W={window} cap={cap} aux={None if aux is None else aux.shape}"
    kw = dict(softmax_scale=b.softmax_scale, sliding_window=window, logits_soft_cap=cap)
    exact = ragged_decode_exact(*np_args(b), softmax_aux=aux, **kw)
    strict = ragged_decode_strict(*np_args(b), block_size=max(S, 1), softmax_aux=aux, **kw)
    finite = np.isfinite(strict).all(axis=(1, 2))
    for flags in (0, _native.RPA_FLAG_FORCE_GENERIC):
        out = to_np(ragged_decode_attention(*b.args(), None if aux is None else torch.from_numpy(aux).to(DEV), _flags=flags,
                                            **kw))
        assert np.isfinite(out).all(), what
        if finite.any():
            assert_bf16_parity_stepwise(out[finite], strict[finite], f"{what} flags={flags}", exact=exact[finite])
        mx, mean = err_stats(out, exact, n)
        assert mx <= 4e-2 and mean <= 2e-3, f"{what} flags={flags}: vs float64 max-abs {mx:.4g} mean-abs {mean:.4g}"
