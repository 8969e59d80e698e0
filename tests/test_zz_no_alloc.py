"""rpa_fwd_launch_static, the entry point that allocates nothing, against rpa_fwd_launch.

Both run the same kernels; the static one keeps split tickets, queue counters and partial attention states in a
device array inside the library instead of a caller's workspace.  Outputs must agree bit for bit (the kernels are
deterministic), on two calls in a row of which the second is smaller, so that whatever the first call left in the
array -- partial states of more parts, counters -- meets a call that uses less of it.
"""

import numpy as np
import pytest
import torch

from ejkernel_amd import _native
from ejkernel_amd.modules import RaggedPageAttention, RaggedPageAttentionConfig
from ejkernel_amd.workloads import make_batch
from tests.helpers import assert_bf16_parity, run_strict, to_np

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def run(b, static, flags=0):
    out = torch.full_like(b.queries, 7.0)  # allocated by the caller, before the call
    RaggedPageAttention().run(*b.args(), softmax_scale=b.softmax_scale, logits_soft_cap=b.logits_soft_cap,
                              sliding_window=b.sliding_window, cfg=RaggedPageAttentionConfig(), _flags=flags,
                              _out=out, _static_scratch=static)
    torch.cuda.synchronize()
    return out


def batches():
    # few long sequences: every (sequence, kv head) is split over many wavefronts, whose partial states go through
    # the scratch; then a smaller batch of the same kind; then a mixed batch whose prefill tiles draw from the queue
    # counters (forced with RPA_FLAG_PREFILL_TILES), and a smaller one again
    big = make_batch([1, 1, 1], [20000, 9000, 14001], num_q_heads=8, num_kv_heads=2, head_dim=128, page_size=16,
                     pages_per_seq=1280, seed=31, device=DEV)
    small = make_batch([1, 2], [3000, 700], num_q_heads=8, num_kv_heads=2, head_dim=128, page_size=16,
                       pages_per_seq=192, seed=32, device=DEV)
    mixed = make_batch([200, 1, 1, 130, 1], [900, 4000, 77, 130, 2500], num_q_heads=8, num_kv_heads=2, head_dim=128,
                       page_size=16, pages_per_seq=256, seed=33, device=DEV, sliding_window=1500)
    mixed_small = make_batch([70, 1], [300, 1200], num_q_heads=8, num_kv_heads=2, head_dim=64, page_size=16,
                             pages_per_seq=128, seed=34, device=DEV, logits_soft_cap=30.0)
    # one long chunk alone: few prefill tiles, whose key ranges are cut and whose parts meet in the scratch; then a shorter one
    chunk = make_batch([300], [2300], num_q_heads=8, num_kv_heads=2, head_dim=128, page_size=16, pages_per_seq=160, seed=35,
                       device=DEV)
    chunk_small = make_batch([130], [900], num_q_heads=8, num_kv_heads=2, head_dim=128, page_size=16, pages_per_seq=64,
                             seed=36, device=DEV)
    tiles = _native.RPA_FLAG_PREFILL_TILES | _native.RPA_FLAG_PLAIN_TILES
    return [(big, 0), (small, 0), (mixed, _native.RPA_FLAG_PREFILL_TILES), (mixed_small, _native.RPA_FLAG_PREFILL_TILES),
            (chunk, tiles), (chunk_small, tiles)]


def test_static_scratch_matches_the_workspace_entry_point_on_consecutive_calls():
    lib = _native.load()
    assert lib.rpa_static_scratch_bytes() == 34 << 20
    cases = batches()
    want = [run(b, False, f) for b, f in cases]
    got = [run(b, True, f) for b, f in cases]  # in a row, each smaller than the one before it within a pair
    for (b, f), w, g in zip(cases, want, got):
        assert torch.equal(w, g), f"static scratch differs from the workspace path (flags {f})"
        rows = b.total_valid_tokens
        assert not g[rows:].any()
    # and the numbers are right, not just equal: the first pair against the restatement of the reference
    for (b, f), g in list(zip(cases, got))[:2]:
        assert_bf16_parity(to_np(g), run_strict(b), b.total_valid_tokens, "static scratch")
    # once more in the opposite order: the small call first, then the large one over its leftovers
    for (b, f), w in reversed(list(zip(cases, want))):
        assert torch.equal(run(b, True, f), w)


def test_static_scratch_rejects_what_does_not_fit():
    """head_dim 256 on the MFMA kernel asks for more scratch than the array holds: a clear error, nothing launched."""
    b = make_batch([1], [100], num_q_heads=16, num_kv_heads=8, head_dim=256, page_size=16, pages_per_seq=16, seed=1,
                   device=DEV)
    with pytest.raises(RuntimeError, match="static scratch"):
        run(b, True)
    # the scalar kernel needs no scratch at all
    g = run(b, True, _native.RPA_FLAG_FORCE_GENERIC)
    assert torch.equal(g, run(b, False, _native.RPA_FLAG_FORCE_GENERIC))


def test_static_entry_point_allocates_nothing_and_replays_from_a_hip_graph():
    """What the entry point is for: a call under HIP graph capture, where nothing may allocate.  After one eager call
    (the first call on a device looks up the scratch array's address) the call is captured, replayed on new queries
    three times with eager work in between, and every replay must equal the eager result of the workspace entry
    point bit for bit.  Across the C call itself neither torch's allocator nor the device's free memory moves."""
    import ctypes

    b = make_batch([1, 1, 1, 3], [9000, 300, 5000, 64], num_q_heads=8, num_kv_heads=2, head_dim=128, page_size=16,
                   pages_per_seq=640, seed=41, device=DEV)
    out = torch.zeros_like(b.queries)
    kw = dict(softmax_scale=b.softmax_scale, cfg=RaggedPageAttentionConfig(), _out=out, _static_scratch=True)
    RaggedPageAttention().run(*b.args(), **kw)   # first call on the device: outside capture
    torch.cuda.synchronize()
    hip = ctypes.CDLL("libamdhip64.so")
    free0, total = ctypes.c_size_t(), ctypes.c_size_t()
    free1 = ctypes.c_size_t()
    assert hip.hipMemGetInfo(ctypes.byref(free0), ctypes.byref(total)) == 0
    allocated, reserved = torch.cuda.memory_allocated(), torch.cuda.memory_reserved()
    RaggedPageAttention().run(*b.args(), **kw)
    torch.cuda.synchronize()
    assert hip.hipMemGetInfo(ctypes.byref(free1), ctypes.byref(total)) == 0
    assert free1.value == free0.value, "device memory moved across rpa_fwd_launch_static"
    assert (torch.cuda.memory_allocated(), torch.cuda.memory_reserved()) == (allocated, reserved)

    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            RaggedPageAttention().run(*b.args(), **kw)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    gen = torch.Generator(device=DEV).manual_seed(5)
    for k in range(3):
        b.queries[: b.total_valid_tokens] = torch.randn(b.total_valid_tokens, 8, 128, device=DEV, generator=gen).to(torch.bfloat16)
        out.fill_(3.0)
        g.replay()
        torch.cuda.synchronize()
        got = out.clone()
        want = run(b, False)   # eager, workspace entry point, allocations and synchronisation between the replays
        assert torch.equal(got, want), f"replay {k} differs from the eager result"
