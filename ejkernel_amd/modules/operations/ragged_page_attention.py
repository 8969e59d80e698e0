"""Ragged paged attention forward: ejkernel's module-level API over the gfx950 HIP library.

The public function keeps the call signature of
``ejkernel/modules/operations/ragged_page_attention.py:540-562`` (seven positional-only
arrays, the rest keyword-only) and the ``RaggedPageAttention`` kernel class keeps the
methods callers touch (``run`` ``:225-318``, ``heuristic_cfg`` ``:320-337``,
``candidate_cfgs`` ``:339-376``).  What the reference does between the two -- an
executor that autotunes over Triton / Pallas / XLA candidates -- has no counterpart:
there is one implementation, reached through ``rpa_fwd_launch`` of
``librpa_mi355x.so``.

Arrays are device tensors (``torch`` tensors on a ROCm device; torch is used for device
memory and streams only).  The op is forward-only: it raises on tensors that require
grad, the same way the reference's native custom call refuses differentiation
(``ejkernel/callib/_triton_call.py:760-799``).
"""

from __future__ import annotations

import ctypes
import threading
import warnings
from typing import Any, Literal

import torch

from ... import _native
from .configs import _PLATFORMS, RaggedPageAttentionConfig

__all__ = ["RaggedPageAttention", "ragged_page_attention"]

_workspaces: dict[tuple[int, int], torch.Tensor] = {}
# (device, stream) pairs kept; the least recently used one goes first.  A workspace is about 35 MB (70 MB at head_dim
# 256) unless ragged_page_attention_v3 keeps the logits of an 8-bit cache between its two launches (up to 2 GiB, 268 MB
# for 256 decode steps over 8192-token block-table rows), so the cache is bounded in bytes as well.
_MAX_WORKSPACES = 16
_MAX_WORKSPACE_BYTES = 4 << 30
_workspaces_lock = threading.Lock()  # host threads launch on streams of their own at the same time
_warned_scalar: set[tuple] = set()   # shapes already reported as running on the scalar kernel


def _compute_mode(compute_dtype: Any) -> int:
    """Map a dtype-like (torch / numpy / jax dtype or its name) to an RPA_COMPUTE_* mode."""
    name = getattr(compute_dtype, "name", None) or getattr(compute_dtype, "__name__", None) or str(compute_dtype)
    name = name.replace("torch.", "").lower()
    if name in ("bfloat16", "bf16"):
        return _native.RPA_COMPUTE_BF16
    if name in ("float32", "f32", "float"):
        return _native.RPA_COMPUTE_F32
    raise ValueError(f"compute_dtype={compute_dtype!r} is not supported (bfloat16 or float32)")


def _static_validate(queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, *,
                     sliding_window, logits_soft_cap, cfg, vmem_limit_bytes):
    """Shape / dtype rules of the reference.

    ``static_validate_inputs``
    (ejkernel/kernels/_pallas/tpu/ragged_page_attention/_pallas_impl_fwd.py:177-230) plus
    the rank and named-dimension checks the jaxtyping decorator performs at the backend
    entry (ejkernel/kernels/_xla/ragged_page_attention/_interface.py:26-47).
    """
    if queries.dim() != 3:
        raise ValueError(f"queries must be [total_tokens, num_q_heads, head_dim], got {tuple(queries.shape)}")
    if kv_pages.dim() != 4:
        raise ValueError(
            f"kv_pages must be [num_pages, page_size, num_combined_kv_heads, head_dim], got {tuple(kv_pages.shape)}"
        )
    if block_tables.dim() != 2:
        raise ValueError(f"block_tables must be [num_seqs, pages_per_seq], got {tuple(block_tables.shape)}")
    _, num_q_heads, head_dim = queries.shape
    _, _, num_combined_kv_heads, head_dim_k = kv_pages.shape
    if num_combined_kv_heads % 2 != 0:
        raise ValueError(f"{num_combined_kv_heads=} must be even (K and V heads interleaved).")
    num_kv_heads = num_combined_kv_heads // 2
    max_num_seqs, pages_per_seq = block_tables.shape
    if isinstance(num_seqs, torch.Tensor) and tuple(num_seqs.shape) != (1,):
        raise ValueError(f"num_seqs.shape={tuple(num_seqs.shape)} must be (1,)")
    if head_dim_k != head_dim:
        raise ValueError(f"Q head_dim {head_dim} must be the same as that of K/V {head_dim_k}.")
    if tuple(context_lens.shape) != (max_num_seqs,):
        raise ValueError(
            f"Expected context_lens.shape={tuple(context_lens.shape)} to be ({max_num_seqs},) where "
            "`max_num_seqs` is `block_tables.shape[0]`."
        )
    if tuple(query_start_loc.shape) != (max_num_seqs + 1,):
        raise ValueError(
            f"Expected query_start_loc.shape={tuple(query_start_loc.shape)} to be ({max_num_seqs + 1},) where "
            "`max_num_seqs` is `block_tables.shape[0]`."
        )
    for name, t in (("context_lens", context_lens), ("block_tables", block_tables),
                    ("query_start_loc", query_start_loc)):
        if t.dtype != torch.int32:
            raise ValueError(f"The dtype of `context_lens`, `block_tables`, and `query_start_loc` must be int32. "
                             f"Got {name}.dtype={t.dtype}.")
    if isinstance(num_seqs, torch.Tensor) and num_seqs.dtype != torch.int32:
        raise ValueError(f"num_seqs.dtype={num_seqs.dtype} must be int32")
    if num_q_heads % num_kv_heads != 0:
        raise ValueError(f"{num_q_heads=} must be divisible by {num_kv_heads=}")
    if sliding_window is not None and sliding_window <= 0:
        raise ValueError(f"{sliding_window=} must be positive.")
    if logits_soft_cap is not None and logits_soft_cap == 0.0:
        raise ValueError(f"{logits_soft_cap=} must not be 0.0.")
    if cfg.num_kv_pages_per_block is not None and not 0 < cfg.num_kv_pages_per_block <= pages_per_seq:
        raise ValueError(f"num_kv_pages_per_block={cfg.num_kv_pages_per_block} must be in range (0, {pages_per_seq}].")
    if cfg.num_queries_per_block is not None and cfg.num_queries_per_block <= 0:
        raise ValueError(f"num_queries_per_block={cfg.num_queries_per_block} must be positive.")
    if vmem_limit_bytes is not None and vmem_limit_bytes <= 0:
        raise ValueError(f"{vmem_limit_bytes=} must be positive.")
    if queries.dtype != kv_pages.dtype:
        raise ValueError(f"queries.dtype={queries.dtype} and kv_pages.dtype={kv_pages.dtype} must match")
    if queries.dtype not in (torch.bfloat16, torch.float32):
        raise ValueError(f"queries.dtype={queries.dtype} is not supported (bfloat16 or float32)")


def _sinks_per_q_head(softmax_aux: torch.Tensor, num_q_heads: int, num_kv_heads: int) -> torch.Tensor:
    """Broadcast sink logits to fp32 ``[num_q_heads, n_sinks]``
    (ejkernel/kernels/_xla/ragged_page_attention/_xla_impl_fwd.py:60-77)."""
    aux = softmax_aux.to(torch.float32)
    group = num_q_heads // num_kv_heads
    if aux.dim() == 2:
        if aux.shape[0] == num_q_heads:
            return aux.contiguous()
        if aux.shape[0] == num_kv_heads:
            return aux.repeat_interleave(group, dim=0).contiguous()
        raise ValueError(
            f"softmax_aux first dim must be num_q_heads ({num_q_heads}) or num_kv_heads ({num_kv_heads}), "
            f"got {tuple(aux.shape)}"
        )
    if aux.dim() == 1:
        return aux[None, :].expand(num_q_heads, aux.shape[0]).contiguous()
    raise ValueError(f"Unsupported softmax_aux shape: {tuple(aux.shape)}")


def _workspace(device: torch.device, nbytes: int, stream_ptr: int) -> torch.Tensor:
    """Workspace of this (device, stream), grown on demand; its counters are cleared once per allocation.

    Launches that share a workspace must not overlap in time, and launches on different streams may: every stream
    gets its own.
    """
    key = (device.index if device.index is not None else torch.cuda.current_device(), int(stream_ptr))
    with _workspaces_lock:
        ws = _workspaces.pop(key, None)  # re-inserted below: the dict keeps its keys in order of last use
        if ws is None or ws.numel() < nbytes:
            # A stream that no longer exists leaves its workspace behind (torch has no hook for a stream's end), so the
            # cache is bounded.  The evicted tensor's memory goes back to torch's caching allocator, which keeps it away
            # from other streams until the work queued on this one has finished.
            want = max(nbytes, 256)
            while _workspaces and (len(_workspaces) >= _MAX_WORKSPACES or
                                   sum(t.numel() for t in _workspaces.values()) + want > _MAX_WORKSPACE_BYTES):
                _workspaces.pop(next(iter(_workspaces)))
            ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=device)
            rc = _native.load().rpa_workspace_init(ctypes.c_void_p(ws.data_ptr()), ws.numel(), ctypes.c_void_p(stream_ptr))
            if rc != 0:
                raise RuntimeError(f"rpa_workspace_init failed ({rc}): {_native.last_error()}")
        _workspaces[key] = ws
    return ws


def _launch(queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, *, softmax_scale,
            logits_soft_cap, compute_dtype, sliding_window, softmax_aux, cfg, flags: int = 0,
            kv_start=None, out=None, static_scratch=False) -> torch.Tensor:
    lib = _native.load()
    if not queries.is_cuda:
        raise RuntimeError(
            "ragged_page_attention needs tensors on a ROCm device (gfx950); there is no CPU implementation in "
            "this package."
        )
    dev = queries.device
    for name, t in (("kv_pages", kv_pages), ("context_lens", context_lens), ("block_tables", block_tables),
                    ("query_start_loc", query_start_loc)):
        if t.device != dev:
            raise ValueError(f"{name} is on {t.device}, queries on {dev}")
    if any(t.requires_grad for t in (queries, kv_pages)):
        raise NotImplementedError("ragged_page_attention is forward-only; detach the inputs")

    total_tokens, num_q_heads, head_dim = queries.shape
    num_pages, page_size, num_combined, _ = kv_pages.shape
    num_kv_heads = num_combined // 2
    max_num_seqs, pages_per_seq = block_tables.shape
    if softmax_scale is None:  # _interface.py:94-95
        softmax_scale = head_dim**-0.5

    queries = queries.contiguous()
    kv_pages = kv_pages.contiguous()
    context_lens = context_lens.contiguous()
    block_tables = block_tables.contiguous()
    query_start_loc = query_start_loc.contiguous()
    if isinstance(num_seqs, torch.Tensor):
        num_seqs_t = num_seqs.to(device=dev).contiguous()
    else:
        num_seqs_t = torch.tensor([int(num_seqs)], dtype=torch.int32, device=dev)
    sinks = None
    if softmax_aux is not None:
        sinks = _sinks_per_q_head(softmax_aux.to(dev), num_q_heads, num_kv_heads)

    if out is None:
        out = torch.empty_like(queries)
    elif out.shape != queries.shape or out.dtype != queries.dtype or out.device != dev or not out.is_contiguous():
        raise ValueError("out must be a contiguous tensor of the shape, dtype and device of queries")
    p = _native.RpaParams()
    p.queries = queries.data_ptr()
    p.kv_pages = kv_pages.data_ptr()
    p.context_lens = context_lens.data_ptr()
    p.block_tables = block_tables.data_ptr()
    p.query_start_loc = query_start_loc.data_ptr()
    p.num_seqs = num_seqs_t.data_ptr()
    p.sinks = sinks.data_ptr() if sinks is not None else None
    p.out = out.data_ptr()
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = total_tokens, num_q_heads, num_kv_heads, head_dim
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = page_size, num_pages, max_num_seqs, pages_per_seq
    p.num_sinks = 0 if sinks is None else sinks.shape[1]
    p.softmax_scale = float(softmax_scale)
    p.logits_soft_cap = 0.0 if logits_soft_cap is None else float(logits_soft_cap)
    p.sliding_window = 0 if sliding_window is None else int(sliding_window)
    p.dtype = _native.RPA_DTYPE_BF16 if queries.dtype == torch.bfloat16 else _native.RPA_DTYPE_F32
    p.compute = _compute_mode(compute_dtype)
    p.num_queries_per_block = cfg.num_queries_per_block or 0
    p.num_kv_pages_per_block = cfg.num_kv_pages_per_block or 0
    p.num_warps = cfg.num_warps or 0
    p.num_stages = cfg.num_stages or 0
    p.flags = flags
    if kv_start is not None:  # first visible key per sequence (RpaParams.kv_start); not a parameter of the reference op
        kv_start = kv_start.to(device=dev, dtype=torch.int32).contiguous()
        p.kv_start = kv_start.data_ptr()

    if p.dtype == _native.RPA_DTYPE_BF16 and p.compute == _native.RPA_COMPUTE_BF16 and not (flags & _native.RPA_FLAG_FORCE_GENERIC):
        # a bf16 call is expected on the MFMA kernels: say so, once per shape, when it is not
        shape = (head_dim, page_size, max_num_seqs)
        if shape not in _warned_scalar and lib.rpa_kernel_path(ctypes.byref(p)) == 0:
            _warned_scalar.add(shape)
            warnings.warn(
                f"ragged_page_attention: head_dim={head_dim}, page_size={page_size}, max_num_seqs={max_num_seqs} runs on "
                "the scalar kernel (exact, about fifty times slower on a decode batch): the MFMA kernels take head_dim "
                "64..256 in multiples of 16, page sizes that are powers of two from 4 and up to 16384 sequences",
                RuntimeWarning, stacklevel=3)
    with torch.cuda.device(dev):
        stream_ptr = torch.cuda.current_stream(dev).cuda_stream
        if static_scratch:  # the entry point that allocates nothing: scratch inside the library, no workspace
            rc = lib.rpa_fwd_launch_static(ctypes.byref(p), ctypes.c_void_p(stream_ptr))
        else:
            nbytes = int(lib.rpa_workspace_bytes(ctypes.byref(p)))
            ws = _workspace(dev, nbytes, stream_ptr)
            p.workspace = ws.data_ptr()
            p.workspace_bytes = ws.numel()
            rc = lib.rpa_fwd_launch(ctypes.byref(p), ctypes.c_void_p(stream_ptr))
    if rc != 0:
        msg = _native.last_error()
        if rc == -1:
            raise ValueError(f"rpa_fwd_launch rejected the arguments: {msg}")
        raise RuntimeError(f"rpa_fwd_launch failed ({rc}): {msg}")
    return out


class RaggedPageAttention:
    """Kernel object of the op (ejkernel/modules/operations/ragged_page_attention.py:80-523)."""

    op_id = "ragged_page_attention"

    def __init__(self):
        self.op_id = "ragged_page_attention"

    def get_impl(self, cfg: RaggedPageAttentionConfig):
        """The reference looks a backend up in its registry (``:210-222``); here there is one."""
        cfg.validate()
        return _launch

    def run(
        self,
        queries,
        kv_pages,
        context_lens,
        block_tables,
        query_start_loc,
        num_seqs,
        platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
        softmax_scale: float | None = None,
        logits_soft_cap: float | None = None,
        compute_dtype: Any = torch.bfloat16,
        optimized: bool = False,
        sliding_window: int | None = None,
        softmax_aux=None,
        mask_value: float | None = None,
        vmem_limit_bytes: int | None = None,
        *,
        cfg: RaggedPageAttentionConfig,
        _flags: int = 0,
        _kv_start=None,
        _out=None,
        _static_scratch: bool = False,
    ):
        """Same parameters as the reference's ``run`` (``:225-318``).

        ``platform``, ``optimized``, ``mask_value`` and ``vmem_limit_bytes`` are accepted
        and have no effect, as in the reference's XLA backend (``_interface.py:93``).
        """
        if platform is not None and platform not in _PLATFORMS:
            raise ValueError(f"platform={platform!r} must be one of {_PLATFORMS}")
        del optimized, mask_value
        cfg.validate()
        _static_validate(queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs,
                         sliding_window=sliding_window, logits_soft_cap=logits_soft_cap, cfg=cfg,
                         vmem_limit_bytes=vmem_limit_bytes)
        return _launch(queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs,
                       softmax_scale=softmax_scale, logits_soft_cap=logits_soft_cap, compute_dtype=compute_dtype,
                       sliding_window=sliding_window, softmax_aux=softmax_aux, cfg=cfg, flags=_flags,
                       kv_start=_kv_start, out=_out, static_scratch=_static_scratch)

    def heuristic_cfg(self, inv=None) -> RaggedPageAttentionConfig:
        """Default configuration (``:320-337``)."""
        return RaggedPageAttentionConfig(num_kv_pages_per_block=None, num_queries_per_block=None, num_warps=4,
                                         num_stages=1, platform="auto", backend="any")

    def candidate_cfgs(self, inv=None) -> list[RaggedPageAttentionConfig]:
        """The reference returns autotune candidates (``:339-376``); one kernel, one candidate."""
        return [self.heuristic_cfg(inv)]

    candidate_cfgs_gpu = candidate_cfgs

    def __call__(self, *args, **kwargs):
        kwargs.setdefault("cfg", self.heuristic_cfg())
        return self.run(*args, **kwargs)


def ragged_page_attention(
    queries,
    kv_pages,
    context_lens,
    block_tables,
    query_start_loc,
    num_seqs,
    softmax_aux=None,
    /,
    *,
    softmax_scale: float | None = None,
    logits_soft_cap: float | None = None,
    compute_dtype: Any = torch.bfloat16,
    optimized: bool = False,
    sliding_window: int | None = None,
    mask_value: float | None = None,
    vmem_limit_bytes: int | None = None,
    platform: Literal["triton", "pallas", "cuda", "xla", "auto"] | None = None,
    cfg: RaggedPageAttentionConfig | None = None,
    mesh=None,
    in_specs=None,
    out_specs=None,
):
    """Ragged paged attention forward over a mixed prefill + decode batch.

    Args (ejkernel/modules/operations/ragged_page_attention.py:563-590):
        queries: ``[total_tokens, num_q_heads, head_dim]``, all sequences concatenated.
        kv_pages: ``[num_pages, page_size, 2 * num_kv_heads, head_dim]``; K of kv head ``j``
            at combined index ``2j``, V at ``2j + 1``.
        context_lens: ``[max_num_seqs]`` int32, kv length of each sequence including its
            current query tokens.
        block_tables: ``[max_num_seqs, pages_per_seq]`` int32 physical page per logical page.
        query_start_loc: ``[max_num_seqs + 1]`` int32 cumulative query lengths.
        num_seqs: ``[1]`` int32 tensor (or int), sequences present.
        softmax_aux: optional sink logits ``[num_kv_heads | num_q_heads, n_sinks]`` or ``[n_sinks]``.
        softmax_scale: defaults to ``head_dim ** -0.5``.
        logits_soft_cap: ``cap * tanh(logits / cap)`` before masking.
        compute_dtype: ``bfloat16`` (MFMA path) or ``float32`` (exact path).
        sliding_window: keep keys with ``k_pos > q_pos - window``.
        optimized, mask_value, vmem_limit_bytes, platform: accepted, no effect.
        cfg: tile overrides, see ``RaggedPageAttentionConfig``.
        mesh, in_specs, out_specs: the reference wraps the call in ``shard_map``
            (``:114-208``); this build runs on one GPU and rejects them.

    Returns:
        ``[total_tokens, num_q_heads, head_dim]`` in the dtype of ``queries``; rows at or
        beyond ``query_start_loc[num_seqs]`` are zero.
    """
    if mesh is not None or in_specs is not None or out_specs is not None:
        raise NotImplementedError(
            "mesh/in_specs/out_specs: this build runs on a single GPU; shard sequences or kv heads outside the op"
        )
    return RaggedPageAttention().run(
        queries,
        kv_pages,
        context_lens,
        block_tables,
        query_start_loc,
        num_seqs,
        platform=platform,
        softmax_scale=softmax_scale,
        logits_soft_cap=logits_soft_cap,
        compute_dtype=compute_dtype,
        optimized=optimized,
        sliding_window=sliding_window,
        softmax_aux=softmax_aux,
        mask_value=mask_value,
        vmem_limit_bytes=vmem_limit_bytes,
        cfg=cfg if cfg is not None else RaggedPageAttentionConfig(),
    )
