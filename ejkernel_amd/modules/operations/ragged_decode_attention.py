"""Ragged decode attention: one query token per sequence over contiguous K / V of ``[batch, seq_len, kv heads, D]``.

Module-level API of ``ejkernel/modules/operations/ragged_decode_attention.py`` (six
positional-only arrays -- ``softmax_aux`` the sixth -- and keyword-only options) and the
``RaggedDecodeAttention`` kernel class (``run`` ``:118-133``, ``heuristic_cfg`` ``:186-206``)
over ``rpa_ragged_decode_launch`` of ``librpa_mi355x.so``.  The program it replaces is the
reference's XLA backend, ``ejkernel/kernels/_xla/ragged_decode_attention/_interface.py:26-121``
and ``_xla_impl_fwd.py:25-364``.

Sequence ``b`` attends from position ``sequence_end[b] - 1`` to the keys ``k`` with
``sequence_start[b] <= k < sequence_end[b]`` and, with ``sliding_window=(left, right)``,
``k >= sequence_end[b] - 1 - left`` (no key lies to the right of the query position, so any
``right >= 0`` changes nothing).

Differences from the reference's XLA program, all in its disfavour: it returns NaN when a
sequence's first KV block holds no visible key, and its block recurrence only equals attention
for sequences that fit one KV block (``oracle/ragged_decode_oracle.py`` restates both); this
implementation computes attention in every case and zeros when nothing is visible.

``softmax_aux`` (attention sinks) follows that program too (``_xla_impl_fwd.py:71-75, :98-134``):
with ``num_sinks`` entries per row, the keys ``[sequence_start[b], sequence_start[b] + num_sinks)``
are visible whatever ``sequence_end`` and the window say, and a key at absolute position
``t < num_sinks`` has ``softmax_aux[row, t]`` added to its logit after the soft cap.  A
one-dimensional ``softmax_aux`` serves every head; a two-dimensional one needs 1 row or
``num_q_heads // num_kv_heads`` rows (row ``g`` for the ``g``-th query head of every kv head),
the only shapes the program's broadcast accepts -- any other row count raises ``ValueError`` here,
where the reference fails while tracing.
"""

from __future__ import annotations

import ctypes
from typing import Literal

import torch

from ... import _native
from .configs import _PLATFORMS, FwdParams, RaggedDecodeAttentionConfig
from .ragged_page_attention import _workspace

__all__ = ["RaggedDecodeAttention", "ragged_decode_attention"]


def _static_validate(query, key, value, sequence_start, sequence_end, sliding_window, logits_soft_cap):
    """Ranks and named dimensions of the typed entry (_interface.py:28-37)."""
    if query.dim() != 3:
        raise ValueError(f"query must be [batch, num_q_heads, head_dim], got {tuple(query.shape)}")
    if key.dim() != 4 or tuple(value.shape) != tuple(key.shape):
        raise ValueError("key and value must both be [batch, seq_len, num_kv_heads, head_dim]")
    batch, num_q_heads, head_dim = query.shape
    if key.shape[0] != batch or key.shape[3] != head_dim:
        raise ValueError("key / value disagree with query on batch or head_dim")
    if num_q_heads % key.shape[2] != 0:
        raise ValueError("num_q_heads must be divisible by num_kv_heads")
    for name, t in (("sequence_start", sequence_start), ("sequence_end", sequence_end)):
        if t.dim() != 1 or t.shape[0] != batch or t.dtype != torch.int32:
            raise ValueError(f"{name} must be int32 of shape [batch]")
    if not (query.dtype == key.dtype == value.dtype) or query.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("query, key and value must share one dtype (bfloat16 or float32)")
    if sliding_window is not None:
        if len(sliding_window) != 2 or sliding_window[0] < 0 or sliding_window[1] < 0:
            raise ValueError("sliding_window must be a (left, right) pair of non-negative sizes")
    if logits_soft_cap is not None and logits_soft_cap == 0.0:
        raise ValueError("logits_soft_cap must not be 0")


def _validate_aux(softmax_aux, group: int):
    """``softmax_aux`` as float32 ``[rows, num_sinks]`` with rows in (1, group) (``_xla_impl_fwd.py:118-134``)."""
    if softmax_aux.dim() == 1:
        aux = softmax_aux[None, :]
    elif softmax_aux.dim() == 2:
        aux = softmax_aux
    else:
        raise ValueError(f"softmax_aux must be [num_sinks] or [rows, num_sinks], got {tuple(softmax_aux.shape)}")
    if aux.shape[1] == 0:
        return None
    if aux.shape[0] not in (1, group):
        raise ValueError(
            f"softmax_aux of shape {tuple(softmax_aux.shape)} does not broadcast against the {group} query heads of a "
            "kv head: it needs 1 row or that many"
        )
    if aux.shape[1] > _native.RPA_MAX_SINK_KEYS:
        raise ValueError(f"softmax_aux has {aux.shape[1]} sinks, at most {_native.RPA_MAX_SINK_KEYS} are supported")
    return aux.to(torch.float32).contiguous()


def _launch(query, key, value, sequence_start, sequence_end, *, softmax_scale, sliding_window, logits_soft_cap, cfg,
            flags: int = 0, softmax_aux=None):
    lib = _native.load()
    if not query.is_cuda:
        raise RuntimeError(
            "ragged_decode_attention needs tensors on a ROCm device (gfx950); there is no CPU implementation in this "
            "package."
        )
    dev = query.device
    for name, t in (("key", key), ("value", value), ("sequence_start", sequence_start), ("sequence_end", sequence_end)):
        if t.device != dev:
            raise ValueError(f"{name} is on {t.device}, query on {dev}")
    if any(t.requires_grad for t in (query, key, value)):
        raise NotImplementedError("ragged_decode_attention is forward-only; detach the inputs")
    batch, num_q_heads, head_dim = query.shape
    _, seq_len, num_kv_heads, _ = key.shape
    query, key, value = query.contiguous(), key.contiguous(), value.contiguous()
    sequence_start, sequence_end = sequence_start.contiguous(), sequence_end.contiguous()
    out = torch.empty_like(query)
    p = _native.RpaRaggedDecodeParams()
    p.query, p.key, p.value = query.data_ptr(), key.data_ptr(), value.data_ptr()
    p.sequence_start, p.sequence_end, p.out = sequence_start.data_ptr(), sequence_end.data_ptr(), out.data_ptr()
    p.batch, p.num_q_heads, p.num_kv_heads, p.head_dim, p.seq_len = batch, num_q_heads, num_kv_heads, head_dim, seq_len
    p.softmax_scale = float(softmax_scale)
    p.logits_soft_cap = 0.0 if logits_soft_cap is None else float(logits_soft_cap)
    p.window_left = -1 if sliding_window is None else int(sliding_window[0])
    bf16 = query.dtype == torch.bfloat16
    p.dtype = _native.RPA_DTYPE_BF16 if bf16 else _native.RPA_DTYPE_F32
    p.compute = _native.RPA_COMPUTE_BF16 if bf16 else _native.RPA_COMPUTE_F32
    p.flags = flags
    aux = None
    if softmax_aux is not None:
        if softmax_aux.device != dev:
            raise ValueError(f"softmax_aux is on {softmax_aux.device}, query on {dev}")
        aux = _validate_aux(softmax_aux, num_q_heads // num_kv_heads)
    if aux is not None:
        p.softmax_aux, p.aux_rows, p.num_sinks = aux.data_ptr(), aux.shape[0], aux.shape[1]
    with torch.cuda.device(dev):
        stream_ptr = torch.cuda.current_stream(dev).cuda_stream
        nbytes = int(lib.rpa_ragged_decode_workspace_bytes(ctypes.byref(p)))
        ws = _workspace(dev, nbytes, stream_ptr)
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
        rc = lib.rpa_ragged_decode_launch(ctypes.byref(p), ctypes.c_void_p(stream_ptr))
    if rc != 0:
        msg = _native.last_error()
        if rc == -1:
            raise ValueError(f"rpa_ragged_decode_launch rejected the arguments: {msg}")
        raise RuntimeError(f"rpa_ragged_decode_launch failed ({rc}): {msg}")
    return out


class RaggedDecodeAttention:
    """Kernel object of the op (ejkernel/modules/operations/ragged_decode_attention.py:75-400)."""

    op_id = "ragged_decode_attention"

    def __init__(self):
        self.op_id = "ragged_decode_attention"

    def get_impl(self, cfg: RaggedDecodeAttentionConfig):
        """The reference looks a backend up in its registry (``:103-116``); here there is one."""
        cfg.validate()
        return _launch

    def run(
        self,
        query,
        key,
        value,
        sequence_start,
        sequence_end,
        softmax_scale: float | None = None,
        sliding_window: tuple[int, int] | None = None,
        logits_soft_cap: float | None = None,
        softmax_aux=None,
        platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
        *,
        cfg: RaggedDecodeAttentionConfig,
        _flags: int = 0,
    ):
        """Same parameters as the reference's ``run`` (``:118-133``).  A query of ``[batch, 1, heads, D]`` is accepted too."""
        if platform is not None and platform not in _PLATFORMS:
            raise ValueError(f"platform={platform!r} must be one of {_PLATFORMS}")
        cfg.validate()
        squeeze = query.dim() == 4 and query.shape[1] == 1
        q3 = query[:, 0] if squeeze else query
        _static_validate(q3, key, value, sequence_start, sequence_end, sliding_window, logits_soft_cap)
        if softmax_scale is None:  # _xla_impl_fwd.py:333-334
            softmax_scale = 1.0 / (q3.shape[-1] ** 0.5)
        out = _launch(q3, key, value, sequence_start, sequence_end, softmax_scale=softmax_scale,
                      sliding_window=sliding_window, logits_soft_cap=logits_soft_cap, cfg=cfg, flags=_flags,
                      softmax_aux=softmax_aux)
        return out[:, None] if squeeze else out

    def heuristic_cfg(self, inv=None) -> RaggedDecodeAttentionConfig:
        """Default configuration (``:186-206``): the block sizes are carried, the kernel picks its own."""
        return RaggedDecodeAttentionConfig(
            fwd_params=FwdParams(blocksize_heads=16, num_key_splits=16, kv_blocksize=128, num_warps=4, num_stages=2),
            platform="auto", backend="any")

    def candidate_cfgs(self, inv=None):
        return [self.heuristic_cfg(inv)]


_kernel = RaggedDecodeAttention()


def ragged_decode_attention(
    query,
    key,
    value,
    sequence_start,
    sequence_end,
    softmax_aux=None,
    /,
    *,
    softmax_scale: float | None = None,
    sliding_window: tuple[int, int] | None = None,
    logits_soft_cap: float | None = None,
    platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
    cfg: RaggedDecodeAttentionConfig | None = None,
    mesh=None,
    in_specs=None,
    out_specs=None,
    _flags: int = 0,
):
    """Signature of the reference's ``ragged_decode_attention``; returns ``[batch, num_q_heads, head_dim]``."""
    if mesh is not None or in_specs is not None or out_specs is not None:
        raise NotImplementedError("sharded execution (mesh / in_specs / out_specs) is not part of this build: one GPU")
    if cfg is None:
        cfg = _kernel.heuristic_cfg()
    return _kernel.run(query, key, value, sequence_start, sequence_end, softmax_scale, sliding_window, logits_soft_cap,
                       softmax_aux, platform, cfg=cfg, _flags=_flags)
