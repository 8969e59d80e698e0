"""Ragged paged attention v3: write the new tokens' K/V into the paged cache, then attend.

Module-level API of ``ejkernel/modules/operations/ragged_page_attention_v3.py:787-812``
(eight positional-only arrays, the rest keyword-only; returns ``(output, kv_cache)``) and
the ``RaggedPageAttentionv3`` kernel class (``run`` ``:377-397``, ``heuristic_cfg``
``:659-679``) over ``rpa_v3_launch`` of ``librpa_mi355x.so``.  The program it replaces is
``ejkernel/kernels/_xla/ragged_page_attention_v3/_kernel.py:127-318``.

The cache is updated in place and returned (the reference donates it,
``_kernel.py:124``).  Its five-dimensional layout
``[num_pages, page_size, 2 * num_kv_heads / packing, packing, head_dim_padded]`` is, for a
head_dim that is a multiple of 128 and an even combined-head count, byte for byte the
``[num_pages, page_size, 2 * num_kv_heads, head_dim]`` layout of the v2 operation.  A head_dim
that is no multiple of 128 has its rows padded to one (``merge_kv``, ``_kernel.py:44-57``): the
kernels then walk the cache with the row pitch of the padded rows and neither read nor write
the padding.  The same holds for a combined-head count padded to a multiple of the packing
(an odd ``num_kv_heads`` under an 8-bit cache).

``distribution[-1]`` is the number of sequences (``_kernel.py:195``).

Cache dtypes: the dtype of the queries (bfloat16 or float32), or ``torch.float8_e4m3fn`` /
``torch.float8_e5m2`` with bfloat16 queries (keys and values then come in the same 8-bit
type, as the reference's ``merge_kv`` demands; packing 4).  With an 8-bit cache the program's
casts apply: ``Q / q_scale`` is clipped to the type's finite range and cast to it when
``q_scale`` is given (``_kernel.py:249-254``), and the normalised probabilities are cast to it
(``:279``), so in e4m3 probabilities below 2**-10 count as zero (2**-17 in e5m2).
"""

from __future__ import annotations

import ctypes
from typing import Literal

import torch

from ... import _native
from .configs import _PLATFORMS, RaggedPageAttentionv3Config
from .ragged_page_attention import _workspace

__all__ = ["RaggedPageAttentionv3", "ragged_page_attention_v3"]

# 8-bit cache dtypes (the OCP formats; the fnuz variants are other encodings and are not accepted)
_FP8 = {torch.float8_e4m3fn: _native.RPA_DTYPE_FP8_E4M3, torch.float8_e5m2: _native.RPA_DTYPE_FP8_E5M2}


def _packing(dtype: torch.dtype) -> int:
    return 32 // (torch.finfo(dtype).bits)


def _static_validate(q, k, v, kv_cache, kv_lens, block_tables, query_start_loc, distribution, *, sliding_window,
                     logits_soft_cap):
    """``static_validate_inputs`` (_kernel.py:71-120) and the shapes the backend entry checks (_interface.py:27-36)."""
    if not (q.dim() == k.dim() == v.dim() == 3):
        raise ValueError("q,k,v must be 3D")
    if k.shape != v.shape or q.shape[0] != k.shape[0] or q.shape[2] != k.shape[2]:
        raise ValueError("shape mismatch among q,k,v")
    _, hq, d = q.shape
    hkv = k.shape[1]
    if hq % hkv != 0:
        raise ValueError("num_q_heads must be divisible by num_kv_heads")
    if kv_cache.dim() != 5:
        raise ValueError("kv_cache must be [num_pages, page_size, num_kv_heads_x2 / packing, packing, head_dim_padded]")
    _, page_size, hx2_per_pack, pack, dalign = kv_cache.shape
    if dalign != -(-d // 128) * 128:
        raise ValueError("cache last dim must be align_to(D,128)")
    if not kv_cache.dtype.is_floating_point:
        raise ValueError("kv_cache must be float")
    if pack != _packing(kv_cache.dtype):
        raise ValueError("packing mismatch")
    for t in (kv_lens, block_tables, query_start_loc, distribution):
        if t.dtype != torch.int32:
            raise ValueError("index arrays must be int32")
    if kv_lens.dim() != 1 or block_tables.dim() != 1:
        raise ValueError("kv_lens and block_tables must be 1D")
    max_num_seqs = kv_lens.shape[0]
    if block_tables.numel() % max_num_seqs != 0:
        raise ValueError("block_tables size % num_seqs != 0")
    if tuple(query_start_loc.shape) != (max_num_seqs + 1,):
        raise ValueError("query_start_loc bad shape")
    if tuple(distribution.shape) != (3,):
        raise ValueError("distribution shape must be (3,)")
    if page_size % pack != 0:
        raise ValueError("page_size must be divisible by packing")
    if sliding_window is not None and sliding_window <= 0:
        raise ValueError("sliding_window > 0")
    if logits_soft_cap is not None and logits_soft_cap == 0.0:
        raise ValueError("soft_cap != 0")
    # limits of this implementation
    if hx2_per_pack != -(-2 * hkv // pack):
        raise ValueError("cache dim 2 must be cdiv(2 * num_kv_heads, packing)")
    if not (k.dtype == v.dtype == kv_cache.dtype):
        raise ValueError("keys, values and kv_cache must share one dtype")  # merge_kv asserts it, the update needs it
    if kv_cache.dtype in _FP8:
        if q.dtype != torch.bfloat16:
            raise ValueError("an 8-bit cache takes bfloat16 queries")
    elif q.dtype != kv_cache.dtype or q.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError("queries, keys, values and kv_cache must share one dtype (bfloat16 or float32), or the cache "
                         "(with keys and values) is float8_e4m3fn or float8_e5m2 and the queries bfloat16; other "
                         "cache types are not built")


def _launch(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution, *, softmax_scale,
            sliding_window, logits_soft_cap, q_scale, k_scale, v_scale, cfg, flags: int = 0):
    lib = _native.load()
    if not queries.is_cuda:
        raise RuntimeError(
            "ragged_page_attention_v3 needs tensors on a ROCm device (gfx950); there is no CPU implementation in "
            "this package."
        )
    dev = queries.device
    for name, t in (("keys", keys), ("values", values), ("kv_cache", kv_cache), ("kv_lens", kv_lens),
                    ("block_tables", block_tables), ("query_start_loc", query_start_loc), ("distribution", distribution)):
        if t.device != dev:
            raise ValueError(f"{name} is on {t.device}, queries on {dev}")
    if any(t.requires_grad for t in (queries, keys, values, kv_cache)):
        raise NotImplementedError("ragged_page_attention_v3 is forward-only; detach the inputs")
    if not kv_cache.is_contiguous():
        raise ValueError("kv_cache must be contiguous: it is updated in place")
    for name, sc in (("q_scale", q_scale), ("k_scale", k_scale), ("v_scale", v_scale)):
        if sc is not None and not sc > 0:
            raise ValueError(f"{name}={sc} must be positive")

    total_tokens, num_q_heads, head_dim = queries.shape
    num_kv_heads = keys.shape[1]
    num_pages, page_size = kv_cache.shape[0], kv_cache.shape[1]
    max_num_seqs = kv_lens.shape[0]
    pages_per_seq = block_tables.numel() // max_num_seqs
    queries, keys, values = queries.contiguous(), keys.contiguous(), values.contiguous()
    kv_lens, block_tables = kv_lens.contiguous(), block_tables.contiguous()
    query_start_loc, distribution = query_start_loc.contiguous(), distribution.contiguous()

    out = torch.empty_like(queries)
    v3 = _native.RpaV3Params()
    p = v3.attn
    p.queries = queries.data_ptr()
    p.kv_pages = kv_cache.data_ptr()
    p.context_lens = kv_lens.data_ptr()
    p.block_tables = block_tables.data_ptr()
    p.query_start_loc = query_start_loc.data_ptr()
    p.num_seqs = distribution.data_ptr() + 2 * 4  # distribution[-1]
    p.sinks = None
    p.out = out.data_ptr()
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = total_tokens, num_q_heads, num_kv_heads, head_dim
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = page_size, num_pages, max_num_seqs, pages_per_seq
    p.num_sinks = 0
    p.softmax_scale = float(softmax_scale)
    p.logits_soft_cap = 0.0 if logits_soft_cap is None else float(logits_soft_cap)
    p.sliding_window = 0 if sliding_window is None else int(sliding_window)
    bf16 = queries.dtype == torch.bfloat16
    p.dtype = _native.RPA_DTYPE_BF16 if bf16 else _native.RPA_DTYPE_F32
    p.compute = _native.RPA_COMPUTE_BF16 if bf16 else _native.RPA_COMPUTE_F32
    p.num_queries_per_block = cfg.num_queries_per_block or 0
    p.num_kv_pages_per_block = cfg.num_kv_pages_per_block or 0
    p.num_warps = cfg.num_warps or 0
    p.num_stages = cfg.num_stages or 0
    p.flags = flags | _native.RPA_FLAG_FP32_LOGITS
    p.q_scale = 0.0 if q_scale is None else float(q_scale)
    p.k_scale = 0.0 if k_scale is None else float(k_scale)
    p.v_scale = 0.0 if v_scale is None else float(v_scale)
    v3.new_keys = keys.data_ptr()
    v3.new_values = values.data_ptr()
    v3.cache_dtype = _FP8.get(kv_cache.dtype, p.dtype)
    v3.cache_head_dim = kv_cache.shape[4]
    v3.cache_combined_heads = kv_cache.shape[2] * kv_cache.shape[3]
    v3.reserved = 0

    with torch.cuda.device(dev):
        stream_ptr = torch.cuda.current_stream(dev).cuda_stream
        nbytes = int(lib.rpa_v3_workspace_bytes(ctypes.byref(v3)))
        ws = _workspace(dev, nbytes, stream_ptr)
        p.workspace = ws.data_ptr()
        p.workspace_bytes = ws.numel()
        rc = lib.rpa_v3_launch(ctypes.byref(v3), ctypes.c_void_p(stream_ptr))
    if rc != 0:
        msg = _native.last_error()
        if rc == -1:
            raise ValueError(f"rpa_v3_launch rejected the arguments: {msg}")
        raise RuntimeError(f"rpa_v3_launch failed ({rc}): {msg}")
    return out, kv_cache


class RaggedPageAttentionv3:
    """Kernel object of the op (ejkernel/modules/operations/ragged_page_attention_v3.py:188-785)."""

    op_id = "ragged_page_attention_v3"

    def __init__(self):
        self.op_id = "ragged_page_attention_v3"

    def get_impl(self, cfg: RaggedPageAttentionv3Config):
        """The reference looks a backend up in its registry (``:362-375``); here there is one."""
        cfg.validate()
        return _launch

    def run(
        self,
        queries,
        keys,
        values,
        kv_cache,
        kv_lens,
        block_tables,
        query_start_loc,
        distribution,
        softmax_scale: float = 1.0,
        sliding_window: int | None = None,
        logits_soft_cap: float | None = None,
        q_scale: float | None = None,
        k_scale: float | None = None,
        v_scale: float | None = None,
        vmem_limit_bytes: int | None = None,
        *,
        platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
        cfg: RaggedPageAttentionv3Config,
        _flags: int = 0,
    ):
        """Same parameters as the reference's ``run`` (``:377-397``); ``platform`` and ``vmem_limit_bytes`` have no effect."""
        if platform is not None and platform not in _PLATFORMS:
            raise ValueError(f"platform={platform!r} must be one of {_PLATFORMS}")
        del vmem_limit_bytes
        cfg.validate()
        _static_validate(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution,
                         sliding_window=sliding_window, logits_soft_cap=logits_soft_cap)
        if softmax_scale is None:  # _interface.py:74-75
            softmax_scale = queries.shape[-1] ** -0.5
        return _launch(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution,
                       softmax_scale=softmax_scale, sliding_window=sliding_window, logits_soft_cap=logits_soft_cap,
                       q_scale=q_scale, k_scale=k_scale, v_scale=v_scale, cfg=cfg, flags=_flags)

    def heuristic_cfg(self, inv=None) -> RaggedPageAttentionv3Config:
        """Default configuration (``:659-679``); the block sizes are chosen on the device, so they stay ``None``."""
        return RaggedPageAttentionv3Config(num_kv_pages_per_block=None, num_queries_per_block=None, num_warps=4,
                                           num_stages=1, platform="auto", backend="any")

    def candidate_cfgs(self, inv=None):
        """One implementation, one candidate (the reference enumerates block-size pairs, ``:681-707``)."""
        return [self.heuristic_cfg(inv)]


_kernel = RaggedPageAttentionv3()


def ragged_page_attention_v3(
    queries,
    keys,
    values,
    kv_cache,
    kv_lens,
    block_tables,
    query_start_loc,
    distribution,
    /,
    *,
    softmax_scale: float = 1.0,
    sliding_window: int | None = None,
    logits_soft_cap: float | None = None,
    q_scale: float | None = None,
    k_scale: float | None = None,
    v_scale: float | None = None,
    vmem_limit_bytes: int | None = None,
    platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
    cfg: RaggedPageAttentionv3Config | None = None,
    mesh=None,
    in_specs=None,
    out_specs=None,
    _flags: int = 0,
):
    """Signature of ``ragged_page_attention_v3`` (``:787-812``); returns ``(output, kv_cache)``, the cache updated in place."""
    if mesh is not None or in_specs is not None or out_specs is not None:
        raise NotImplementedError("sharded execution (mesh / in_specs / out_specs) is not part of this build: one GPU")
    if cfg is None:
        cfg = _kernel.heuristic_cfg()
    return _kernel.run(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution,
                       softmax_scale, sliding_window, logits_soft_cap, q_scale, k_scale, v_scale, vmem_limit_bytes,
                       platform=platform, cfg=cfg, _flags=_flags)
