"""JAX entry points: the ops as XLA FFI custom calls (``jax.ffi``) over ``librpa_mi355x.so``.

Importing this module needs JAX with a ROCm backend.  It compiles ``csrc/rpa_xla_ffi.cc``
against the FFI headers inside jaxlib (``jax.ffi.include_dir()``), registers the handlers
for platform ``"ROCM"`` and exposes ``ragged_page_attention`` with the reference's
signature (ejkernel/modules/operations/ragged_page_attention.py:540-562), plus
``ragged_page_attention_v3`` (cache donated and returned, as the reference's jitted program does,
ejkernel/kernels/_xla/ragged_page_attention_v3/_kernel.py:110-126), ``page_attention`` and
``ragged_decode_attention``, all traceable under ``jax.jit``.  Like the reference's native call
(ejkernel/callib/_triton_call.py:760-799) they are forward-only: no JVP and no batching rule.

Scratch memory belongs to XLA: every call declares one more result than the op has, ``uint8[n]`` with ``n`` from
the library's ``rpa_*_workspace_bytes`` for the call's static shapes, and drops it; the handlers allocate nothing.

This image has no JAX, so this module has not been built or run here; the torch-tensor
entry point in ``ejkernel_amd.modules`` is the tested one.  Both go through the same C ABI.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import jax
import jax.numpy as jnp
import numpy as np

from . import _native
from .build import HIPCC_FLAGS, LIB_DIR, _hipcc
from .modules.operations.configs import RaggedPageAttentionConfig

_FFI_LIB = LIB_DIR / "librpa_mi355x_xla_ffi.so"
_TARGET = "mi355x_rpa_fwd"
_TARGETS = {_TARGET: "RpaFwd", "mi355x_rpa_v3": "RpaV3", "mi355x_page_attention": "RpaPageAttn",
            "mi355x_ragged_decode_attention": "RpaRaggedDecode"}
_registered = False


def build_ffi() -> Path:
    src = Path(__file__).resolve().parent / "csrc" / "rpa_xla_ffi.cc"
    cmd = [_hipcc(), *HIPCC_FLAGS, "-x", "hip", "-shared", f"-I{jax.ffi.include_dir()}", str(src),
           f"-L{LIB_DIR}", "-lrpa_mi355x", f"-Wl,-rpath,{LIB_DIR}", "-o", str(_FFI_LIB)]
    subprocess.run(cmd, check=True)
    return _FFI_LIB


def _register():
    global _registered
    if _registered:
        return
    _native.load()
    if not _FFI_LIB.exists():
        build_ffi()
    lib = ctypes.CDLL(str(_FFI_LIB))
    for target, symbol in _TARGETS.items():
        jax.ffi.register_ffi_target(target, jax.ffi.pycapsule(getattr(lib, symbol)), platform="ROCM")
    _registered = True


def _scratch(nbytes: int):
    """The extra result every handler takes: the op's workspace, owned and placed by XLA."""
    return jax.ShapeDtypeStruct((max(int(nbytes), 256),), jnp.uint8)


def _rpa_dims(total_tokens, num_q_heads, num_kv_heads, head_dim, page_size, num_pages, max_num_seqs, pages_per_seq, dtype,
              cfg=None, flags=0):
    """RpaParams carrying the static shapes only (what the workspace-size queries read)."""
    p = _native.RpaParams()
    p.total_tokens, p.num_q_heads, p.num_kv_heads, p.head_dim = total_tokens, num_q_heads, num_kv_heads, head_dim
    p.page_size, p.num_pages, p.max_num_seqs, p.pages_per_seq = page_size, num_pages, max_num_seqs, pages_per_seq
    bf16 = jnp.dtype(dtype) == jnp.bfloat16
    p.dtype = _native.RPA_DTYPE_BF16 if bf16 else _native.RPA_DTYPE_F32
    p.compute = _native.RPA_COMPUTE_BF16 if bf16 else _native.RPA_COMPUTE_F32
    if cfg is not None:
        p.num_queries_per_block = cfg.num_queries_per_block or 0
        p.num_kv_pages_per_block = cfg.num_kv_pages_per_block or 0
    p.flags = flags
    return p


def ragged_page_attention(queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, softmax_aux=None, /,
                          *, softmax_scale=None, logits_soft_cap=None, compute_dtype=jnp.bfloat16, optimized=False,
                          sliding_window=None, mask_value=None, vmem_limit_bytes=None, platform=None, cfg=None,
                          mesh=None, in_specs=None, out_specs=None):
    del optimized, mask_value, vmem_limit_bytes, platform
    if mesh is not None:
        raise NotImplementedError("wrap the call in jax.shard_map outside the op (sequence or kv-head sharding)")
    _register()
    cfg = cfg or RaggedPageAttentionConfig()
    cfg.validate()
    total_tokens, num_q_heads, head_dim = queries.shape
    num_pages, page_size, combined, _ = kv_pages.shape
    max_num_seqs, pages_per_seq = block_tables.shape
    if not isinstance(num_seqs, jax.Array):
        num_seqs = jnp.asarray([num_seqs], dtype=jnp.int32)
    operands = [queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs]
    if softmax_aux is not None:
        aux = jnp.asarray(softmax_aux, jnp.float32)
        if aux.ndim == 1:
            aux = jnp.broadcast_to(aux[None], (num_q_heads, aux.shape[0]))
        elif aux.shape[0] != num_q_heads:
            aux = jnp.repeat(aux, num_q_heads // aux.shape[0], axis=0)
        operands.append(aux)
    dims = _rpa_dims(total_tokens, num_q_heads, combined // 2, head_dim, page_size, num_pages, max_num_seqs, pages_per_seq,
                     queries.dtype, cfg)
    nbytes = _native.load().rpa_workspace_bytes(ctypes.byref(dims))
    call = jax.ffi.ffi_call(_TARGET, (jax.ShapeDtypeStruct(queries.shape, queries.dtype), _scratch(nbytes)))
    out, _ = call(
        *operands,
        softmax_scale=np.float32(head_dim**-0.5 if softmax_scale is None else softmax_scale),
        logits_soft_cap=np.float32(0.0 if logits_soft_cap is None else logits_soft_cap),
        sliding_window=np.int32(0 if sliding_window is None else sliding_window),
        compute=np.int32(_native.RPA_COMPUTE_BF16 if jnp.dtype(compute_dtype) == jnp.bfloat16 else _native.RPA_COMPUTE_F32),
        num_queries_per_block=np.int32(cfg.num_queries_per_block or 0),
        num_kv_pages_per_block=np.int32(cfg.num_kv_pages_per_block or 0),
        num_warps=np.int32(cfg.num_warps or 0),
        num_stages=np.int32(cfg.num_stages or 0),
    )
    return out


def ragged_page_attention_v3(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution, /, *,
                             softmax_scale=None, sliding_window=None, logits_soft_cap=None, q_scale=None, k_scale=None,
                             v_scale=None):
    """Cache update + attention; returns ``(out, kv_cache)`` with the cache updated in place (operand 3 is aliased to
    the second result, so jit the caller with the cache donated as the reference does)."""
    _register()
    v = _native.RpaV3Params()
    v.attn = _rpa_dims(queries.shape[0], queries.shape[1], keys.shape[1], queries.shape[2], kv_cache.shape[1], kv_cache.shape[0],
                       kv_lens.shape[0], block_tables.size // max(kv_lens.shape[0], 1), queries.dtype,
                       flags=_native.RPA_FLAG_FP32_LOGITS)
    cache_dt = jnp.dtype(kv_cache.dtype)
    v.cache_dtype = {jnp.dtype(jnp.bfloat16): _native.RPA_DTYPE_BF16, jnp.dtype(jnp.float32): _native.RPA_DTYPE_F32,
                     jnp.dtype(jnp.float8_e4m3fn): _native.RPA_DTYPE_FP8_E4M3,
                     jnp.dtype(jnp.float8_e5m2): _native.RPA_DTYPE_FP8_E5M2}[cache_dt]
    v.cache_head_dim, v.cache_combined_heads = kv_cache.shape[4], kv_cache.shape[2] * kv_cache.shape[3]
    nbytes = _native.load().rpa_v3_workspace_bytes(ctypes.byref(v))
    call = jax.ffi.ffi_call(
        "mi355x_rpa_v3",
        (jax.ShapeDtypeStruct(queries.shape, queries.dtype), jax.ShapeDtypeStruct(kv_cache.shape, kv_cache.dtype), _scratch(nbytes)),
        input_output_aliases={3: 1},
    )
    f32 = lambda x: np.float32(0.0 if x is None else x)  # noqa: E731
    return call(queries, keys, values, kv_cache, kv_lens, block_tables, query_start_loc, distribution,
                softmax_scale=np.float32(queries.shape[-1] ** -0.5 if softmax_scale is None else softmax_scale),
                logits_soft_cap=f32(logits_soft_cap), q_scale=f32(q_scale), k_scale=f32(k_scale), v_scale=f32(v_scale),
                sliding_window=np.int32(0 if sliding_window is None else sliding_window))[:2]


def page_attention(query, key_cache, value_cache, context_lens, block_tables, /, *, attn_scale=None):
    """One query token per sequence over separate paged K and V caches ``[blocks, kv heads, block, head_dim]``."""
    _register()
    p = _native.RpaPageAttnParams()
    p.num_seqs, p.num_q_heads, p.head_dim = query.shape
    p.num_blocks, p.num_kv_heads, p.block_size = key_cache.shape[:3]
    p.max_blocks = block_tables.shape[1]
    bf16 = jnp.dtype(query.dtype) == jnp.bfloat16
    p.dtype = _native.RPA_DTYPE_BF16 if bf16 else _native.RPA_DTYPE_F32
    p.compute = _native.RPA_COMPUTE_BF16 if bf16 else _native.RPA_COMPUTE_F32
    nbytes = _native.load().rpa_page_attention_workspace_bytes(ctypes.byref(p))
    call = jax.ffi.ffi_call("mi355x_page_attention", (jax.ShapeDtypeStruct(query.shape, query.dtype), _scratch(nbytes)))
    return call(query, key_cache, value_cache, context_lens, block_tables,
                attn_scale=np.float32(query.shape[-1] ** -0.5 if attn_scale is None else attn_scale))[0]


def ragged_decode_attention(query, key, value, sequence_start, sequence_end, softmax_aux=None, /, *, softmax_scale=None,
                            logits_soft_cap=None, sliding_window=None):
    """One query token per sequence over contiguous K and V ``[batch, seq_len, kv heads, head_dim]``; ``sliding_window``
    is ``(left, right)`` as in the reference, of which the left part applies to a decode step."""
    _register()
    operands = [query, key, value, sequence_start, sequence_end]
    if softmax_aux is not None:
        aux = jnp.asarray(softmax_aux, jnp.float32)
        operands.append(aux[None] if aux.ndim == 1 else aux)
    p = _native.RpaRaggedDecodeParams()
    p.batch, p.num_q_heads, p.head_dim = query.shape
    p.seq_len, p.num_kv_heads = key.shape[1], key.shape[2]
    bf16 = jnp.dtype(query.dtype) == jnp.bfloat16
    p.dtype = _native.RPA_DTYPE_BF16 if bf16 else _native.RPA_DTYPE_F32
    p.compute = _native.RPA_COMPUTE_BF16 if bf16 else _native.RPA_COMPUTE_F32
    if softmax_aux is not None:
        p.aux_rows, p.num_sinks = operands[-1].shape
    nbytes = _native.load().rpa_ragged_decode_workspace_bytes(ctypes.byref(p))
    call = jax.ffi.ffi_call("mi355x_ragged_decode_attention", (jax.ShapeDtypeStruct(query.shape, query.dtype), _scratch(nbytes)))
    return call(*operands,
                softmax_scale=np.float32(query.shape[-1] ** -0.5 if softmax_scale is None else softmax_scale),
                logits_soft_cap=np.float32(0.0 if logits_soft_cap is None else logits_soft_cap),
                window_left=np.int32(-1 if sliding_window is None else int(sliding_window[0])))[0]
