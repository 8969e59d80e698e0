"""Page attention (one query token per sequence over paged key / value caches).

Module-level API of ``ejkernel/modules/operations/page_attention.py:364-383`` (five
positional-only arrays, the rest keyword-only) and the ``PageAttention`` kernel class
(``run`` ``:128-146``, ``heuristic_cfg`` ``:212-229``, ``candidate_cfgs`` ``:231-247``)
over ``rpa_page_attention_launch`` of ``librpa_mi355x.so``.  The program it replaces is the
reference's XLA backend, ``ejkernel/kernels/_xla/page_attention/_interface.py:25-115`` and
``_xla_impl_fwd.py:22-101``, whose argument handling is kept: ``max_context_len``,
``num_splits != 0``, ``pages_per_compute_block``, ``megacore_mode``,
``inline_seq_dim=False`` and ``attn_logits_soft_cap`` raise ``NotImplementedError``
(``_interface.py:97-108``); ``mask_value`` is accepted and unused.

One difference: a sequence with ``context_lens == 0`` yields zeros here; the reference
program softmaxes a row of equal mask values and returns the mean of whatever the block
table points at.
"""

from __future__ import annotations

import ctypes
from typing import Literal

import torch

from ... import _native
from .configs import _PLATFORMS, PageAttentionConfig
from .ragged_page_attention import _workspace

__all__ = ["PageAttention", "page_attention"]


def _static_validate(query, key_cache, value_cache, context_lens, block_tables):
    """Ranks and named dimensions the reference's typed entry enforces (_interface.py:27-32)."""
    if query.dim() != 3:
        raise ValueError(f"query must be [num_seqs, num_heads, head_dim], got {tuple(query.shape)}")
    if key_cache.dim() != 4 or tuple(value_cache.shape) != tuple(key_cache.shape):
        raise ValueError("key_cache and value_cache must both be [num_blocks, num_kv_heads, block_size, head_dim]")
    if context_lens.dim() != 1 or block_tables.dim() != 2:
        raise ValueError("context_lens must be [num_seqs] and block_tables [num_seqs, max_blocks]")
    num_seqs, num_heads, head_dim = query.shape
    if key_cache.shape[3] != head_dim:
        raise ValueError(f"head_dim of the caches ({key_cache.shape[3]}) differs from the query's ({head_dim})")
    if context_lens.shape[0] != num_seqs or block_tables.shape[0] != num_seqs:
        raise ValueError("context_lens / block_tables disagree with query on num_seqs")
    if num_heads % key_cache.shape[1] != 0:
        raise ValueError("num_heads must be divisible by num_kv_heads")
    if context_lens.dtype != torch.int32 or block_tables.dtype != torch.int32:
        raise ValueError("context_lens and block_tables must be int32")
    if not (query.dtype == key_cache.dtype == value_cache.dtype) or query.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("query and the caches must share one dtype (bfloat16 or float32)")


def _launch(query, key_cache, value_cache, context_lens, block_tables, *, attn_scale, cfg, flags: int = 0):
    lib = _native.load()
    if not query.is_cuda:
        raise RuntimeError(
            "page_attention needs tensors on a ROCm device (gfx950); there is no CPU implementation in this package."
        )
    dev = query.device
    for name, t in (("key_cache", key_cache), ("value_cache", value_cache), ("context_lens", context_lens),
                    ("block_tables", block_tables)):
        if t.device != dev:
            raise ValueError(f"{name} is on {t.device}, query on {dev}")
    if any(t.requires_grad for t in (query, key_cache, value_cache)):
        raise NotImplementedError("page_attention is forward-only; detach the inputs")
    num_seqs, num_heads, head_dim = query.shape
    num_blocks, num_kv_heads, block_size, _ = key_cache.shape
    query, key_cache, value_cache = query.contiguous(), key_cache.contiguous(), value_cache.contiguous()
    context_lens, block_tables = context_lens.contiguous(), block_tables.contiguous()
    out = torch.empty_like(query)
    p = _native.RpaPageAttnParams()
    p.query, p.key_cache, p.value_cache = query.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr()
    p.context_lens, p.block_tables, p.out = context_lens.data_ptr(), block_tables.data_ptr(), out.data_ptr()
    p.num_seqs, p.num_q_heads, p.num_kv_heads, p.head_dim = num_seqs, num_heads, num_kv_heads, head_dim
    p.block_size, p.num_blocks, p.max_blocks = block_size, num_blocks, block_tables.shape[1]
    p.attn_scale = float(attn_scale)
    bf16 = query.dtype == torch.bfloat16
    p.dtype = _native.RPA_DTYPE_BF16 if bf16 else _native.RPA_DTYPE_F32
    p.compute = _native.RPA_COMPUTE_BF16 if bf16 else _native.RPA_COMPUTE_F32
    p.flags = flags
    with torch.cuda.device(dev):
        stream_ptr = torch.cuda.current_stream(dev).cuda_stream
        nbytes = int(lib.rpa_page_attention_workspace_bytes(ctypes.byref(p)))
        ws = _workspace(dev, nbytes, stream_ptr)
        p.workspace, p.workspace_bytes = ws.data_ptr(), ws.numel()
        rc = lib.rpa_page_attention_launch(ctypes.byref(p), ctypes.c_void_p(stream_ptr))
    if rc != 0:
        msg = _native.last_error()
        if rc == -1:
            raise ValueError(f"rpa_page_attention_launch rejected the arguments: {msg}")
        raise RuntimeError(f"rpa_page_attention_launch failed ({rc}): {msg}")
    return out


class PageAttention:
    """Kernel object of the op (ejkernel/modules/operations/page_attention.py:82-362)."""

    op_id = "page_attention"

    def __init__(self):
        self.op_id = "page_attention"

    def get_impl(self, cfg: PageAttentionConfig):
        """The reference looks a backend up in its registry (``:113-126``); here there is one."""
        cfg.validate()
        return _launch

    def run(
        self,
        query,
        key_cache,
        value_cache,
        context_lens,
        block_tables,
        attn_scale: float | None = None,
        max_context_len: int | None = None,
        num_splits: int = 0,
        platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
        *,
        cfg: PageAttentionConfig,
        mask_value: float = -2.381976426469702e38,
        attn_logits_soft_cap: float | None = None,
        pages_per_compute_block: int | None = None,
        megacore_mode: str | None = None,
        inline_seq_dim: bool = True,
        _flags: int = 0,
    ):
        """Same parameters as the reference's ``run`` (``:128-146``), handled as its XLA backend handles them."""
        if platform is not None and platform not in _PLATFORMS:
            raise ValueError(f"platform={platform!r} must be one of {_PLATFORMS}")
        del mask_value
        cfg.validate()
        # _interface.py:97-108
        if max_context_len is not None:
            raise NotImplementedError("max_context_len is not supported in XLA implementation")
        if num_splits != 0:
            raise NotImplementedError("num_splits is not supported in XLA implementation")
        if pages_per_compute_block is not None:
            raise NotImplementedError("pages_per_compute_block is not supported in XLA implementation")
        if megacore_mode is not None:
            raise NotImplementedError("megacore_mode is not supported in XLA implementation")
        if not inline_seq_dim:
            raise NotImplementedError("inline_seq_dim=False is not supported in XLA implementation")
        if attn_logits_soft_cap is not None:
            raise NotImplementedError("attn_logits_soft_cap is not supported in XLA implementation")
        _static_validate(query, key_cache, value_cache, context_lens, block_tables)
        if attn_scale is None:
            # _interface.py:110-111 makes the default scale a float32 array, which promotes the whole computation to
            # float32: q enters unscaled and the logits stay fp32.  (The reference then also returns float32; here
            # the output keeps the query dtype.)  A scale passed as a Python number keeps the query dtype, so q * scale
            # and the logits are rounded to it.
            attn_scale = 1.0 / (query.shape[-1] ** 0.5)
            _flags |= _native.RPA_FLAG_FP32_LOGITS
        return _launch(query, key_cache, value_cache, context_lens, block_tables, attn_scale=attn_scale, cfg=cfg,
                       flags=_flags)

    def heuristic_cfg(self, inv=None) -> PageAttentionConfig:
        """Default configuration (``:212-229``)."""
        return PageAttentionConfig(num_splits=0, pages_per_compute_block=None, num_warps=4, num_stages=1,
                                   platform="auto", backend="any")

    def candidate_cfgs(self, inv=None):
        """No tunable block sizes (``:231-247``)."""
        return []


_kernel = PageAttention()


def page_attention(
    query,
    key_cache,
    value_cache,
    context_lens,
    block_tables,
    /,
    *,
    attn_scale: float | None = None,
    max_context_len: int | None = None,
    num_splits: int = 0,
    mask_value: float = -2.381976426469702e38,
    attn_logits_soft_cap: float | None = None,
    pages_per_compute_block: int | None = None,
    megacore_mode: str | None = None,
    inline_seq_dim: bool = True,
    platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
    cfg: PageAttentionConfig | None = None,
    _flags: int = 0,
):
    """Signature of ``page_attention`` (``:364-383``); returns ``[num_seqs, num_heads, head_dim]``."""
    if cfg is None:
        cfg = _kernel.heuristic_cfg()
    return _kernel.run(query, key_cache, value_cache, context_lens, block_tables, attn_scale, max_context_len,
                       num_splits, platform, cfg=cfg, mask_value=mask_value, attn_logits_soft_cap=attn_logits_soft_cap,
                       pages_per_compute_block=pages_per_compute_block, megacore_mode=megacore_mode,
                       inline_seq_dim=inline_seq_dim, _flags=_flags)
