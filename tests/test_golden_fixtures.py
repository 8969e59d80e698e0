"""Frozen fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py).

They hold outputs of this repository's oracles, not of the reference (which cannot be imported here and ships no
vectors for these operations).  CPU: every oracle still reproduces its fixture bit for bit.  GPU: the device
kernels are held to the frozen outputs within the bf16 tolerance, on both kernel paths.
"""

import os

import numpy as np
import pytest

from oracle import rpa_oracle
from oracle.page_attention_oracle import page_attention_strict
from oracle.ragged_decode_oracle import ragged_decode_strict
from oracle.rpa_oracle import bf16_bits, bf16_from_bits
from oracle.rpa_v3_oracle import rpa_v3

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    with np.load(os.path.join(HERE, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def opt(x):
    return None if float(x) == 0 else (int(x) if np.issubdtype(np.asarray(x).dtype, np.integer) else float(x))


@pytest.mark.parametrize("name", ["rpa_mixed.npz", "rpa_window_cap_d256.npz"])
def test_rpa_oracle_reproduces_its_fixture(name):
    f = load(name)
    out = rpa_oracle.rpa_strict(bf16_from_bits(f["queries"]), bf16_from_bits(f["kv_pages"]), f["context_lens"],
                                f["block_tables"], f["query_start_loc"], f["num_seqs"],
                                softmax_scale=float(f["softmax_scale"]), sliding_window=opt(f["sliding_window"]),
                                logits_soft_cap=opt(f["logits_soft_cap"]))
    assert np.array_equal(bf16_bits(out), f["expected"])


def test_other_oracles_reproduce_their_fixtures():
    f = load("rpa_v3.npz")
    out, new = rpa_v3(*[bf16_from_bits(f[k]) for k in ("queries", "keys", "values", "kv_cache")], f["kv_lens"],
                      f["block_tables"], f["query_start_loc"], f["distribution"], softmax_scale=float(f["softmax_scale"]))
    assert np.array_equal(bf16_bits(out), f["expected"]) and np.array_equal(bf16_bits(new), f["expected_cache"])
    f = load("rpa_v3_e4m3.npz")
    scales = {n: float(f[n]) for n in ("softmax_scale", "q_scale", "k_scale", "v_scale")}
    out, new = rpa_v3(bf16_from_bits(f["queries"]), *[f[k].astype(np.float32) for k in ("keys", "values", "kv_cache")],
                      f["kv_lens"], f["block_tables"], f["query_start_loc"], f["distribution"],
                      cache_dtype="float8_e4m3fn", query_dtype="bfloat16", **scales)
    assert np.array_equal(bf16_bits(out), f["expected"]) and np.array_equal(new, f["expected_cache"].astype(np.float32))
    f = load("page_attention.npz")
    out = page_attention_strict(*[bf16_from_bits(f[k]) for k in ("query", "key_cache", "value_cache")],
                                f["context_lens"], f["block_tables"], attn_scale=float(f["attn_scale"]))
    assert np.array_equal(bf16_bits(out), f["expected"])
    f = load("ragged_decode.npz")
    out = ragged_decode_strict(*[bf16_from_bits(f[k]) for k in ("query", "key", "value")], f["sequence_start"],
                               f["sequence_end"], softmax_scale=float(f["softmax_scale"]), block_size=int(f["block_size"]))
    assert np.array_equal(bf16_bits(out), f["expected"])
    f = load("ragged_decode_sinks.npz")
    out = ragged_decode_strict(*[bf16_from_bits(f[k]) for k in ("query", "key", "value")], f["sequence_start"],
                               f["sequence_end"], softmax_scale=float(f["softmax_scale"]), block_size=int(f["block_size"]),
                               sliding_window=(int(f["window_left"]), 0), softmax_aux=f["softmax_aux"])
    assert np.array_equal(bf16_bits(out), f["expected"])


# ----------------------------------------------------------------------------- device side

def _dev(bits):
    import torch

    return torch.from_numpy(bf16_from_bits(bits)).to(torch.bfloat16).to("cuda:0")


def _idx(a):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).to("cuda:0")


def _check(out, expected_bits, rows, scale=1.0):
    got = out.float().cpu().numpy()[:rows]
    d = np.abs(got - bf16_from_bits(expected_bits)[:rows]) / scale   # scale: what v_scale multiplied the outputs by
    assert d.max() <= 2e-2 and d.mean() <= 2e-3, (d.max(), d.mean())


@pytest.mark.gpu
@pytest.mark.parametrize("flags", [0, 4, 1], ids=["tiled", "tiles", "generic"])
def test_device_kernels_against_the_frozen_outputs(flags):
    from ejkernel_amd.modules import (RaggedPageAttention, RaggedPageAttentionConfig, page_attention,
                                      ragged_decode_attention, ragged_page_attention_v3)

    for name in ("rpa_mixed.npz", "rpa_window_cap_d256.npz"):
        f = load(name)
        out = RaggedPageAttention().run(_dev(f["queries"]), _dev(f["kv_pages"]), _idx(f["context_lens"]),
                                        _idx(f["block_tables"]), _idx(f["query_start_loc"]), _idx(f["num_seqs"]),
                                        softmax_scale=float(f["softmax_scale"]),
                                        sliding_window=opt(f["sliding_window"]),
                                        logits_soft_cap=opt(f["logits_soft_cap"]), cfg=RaggedPageAttentionConfig(),
                                        _flags=flags)
        _check(out, f["expected"], int(f["query_start_loc"][-1]))
    f = load("rpa_v3.npz")
    out, cache = ragged_page_attention_v3(_dev(f["queries"]), _dev(f["keys"]), _dev(f["values"]), _dev(f["kv_cache"]),
                                          _idx(f["kv_lens"]), _idx(f["block_tables"]), _idx(f["query_start_loc"]),
                                          _idx(f["distribution"]), softmax_scale=float(f["softmax_scale"]), _flags=flags)
    _check(out, f["expected"], int(f["query_start_loc"][-1]))
    assert np.array_equal(bf16_bits(cache.float().cpu().numpy()), f["expected_cache"])
    if flags != 1:  # an 8-bit cache runs on the MFMA kernel only
        f = load("rpa_v3_e4m3.npz")
        import torch

        f8 = lambda a: torch.from_numpy(a.astype(np.float32)).to(torch.float8_e4m3fn).to("cuda:0")  # noqa: E731
        scales = {n: float(f[n]) for n in ("softmax_scale", "q_scale", "k_scale", "v_scale")}
        out, cache = ragged_page_attention_v3(_dev(f["queries"]), f8(f["keys"]), f8(f["values"]), f8(f["kv_cache"]),
                                              _idx(f["kv_lens"]), _idx(f["block_tables"]), _idx(f["query_start_loc"]),
                                              _idx(f["distribution"]), _flags=flags, **scales)
        _check(out, f["expected"], int(f["query_start_loc"][-1]), scale=2.0)
        assert np.array_equal(cache.float().cpu().numpy(), f["expected_cache"].astype(np.float32))
    f = load("page_attention.npz")
    out = page_attention(_dev(f["query"]), _dev(f["key_cache"]), _dev(f["value_cache"]), _idx(f["context_lens"]),
                         _idx(f["block_tables"]), attn_scale=float(f["attn_scale"]), _flags=flags)
    _check(out, f["expected"], 4)
    f = load("ragged_decode.npz")
    out = ragged_decode_attention(_dev(f["query"]), _dev(f["key"]), _dev(f["value"]), _idx(f["sequence_start"]),
                                  _idx(f["sequence_end"]), softmax_scale=float(f["softmax_scale"]), _flags=flags)
    _check(out, f["expected"], 4)
    f = load("ragged_decode_sinks.npz")
    out = ragged_decode_attention(_dev(f["query"]), _dev(f["key"]), _dev(f["value"]), _idx(f["sequence_start"]),
                                  _idx(f["sequence_end"]), _idx(f["softmax_aux"]), softmax_scale=float(f["softmax_scale"]),
                                  sliding_window=(int(f["window_left"]), 0), _flags=flags)
    _check(out, f["expected"], 4)
