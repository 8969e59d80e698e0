"""JAX entry point: the op as an XLA FFI custom call (``jax.ffi``) over ``librpa_mi355x.so``.

Importing this module needs JAX with a ROCm backend.  It compiles ``csrc/rpa_xla_ffi.cc``
against the FFI headers inside jaxlib (``jax.ffi.include_dir()``), registers the handler
for platform ``"ROCM"`` and exposes ``ragged_page_attention`` with the reference's
signature (ejkernel/modules/operations/ragged_page_attention.py:540-562), traceable under
``jax.jit``.  Like the reference's native call (ejkernel/callib/_triton_call.py:760-799)
it is forward-only: no JVP and no batching rule.

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
    jax.ffi.register_ffi_target(_TARGET, jax.ffi.pycapsule(lib.RpaFwd), platform="ROCM")
    _registered = True


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
    dims = _native.RpaParams()
    dims.total_tokens, dims.num_q_heads, dims.num_kv_heads, dims.head_dim = total_tokens, num_q_heads, combined // 2, head_dim
    dims.page_size, dims.num_pages, dims.max_num_seqs, dims.pages_per_seq = page_size, num_pages, max_num_seqs, pages_per_seq
    dims.softmax_scale = 1.0
    ws_bytes = int(_native.load().rpa_workspace_bytes(ctypes.byref(dims)))
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
    call = jax.ffi.ffi_call(
        _TARGET,
        (jax.ShapeDtypeStruct(queries.shape, queries.dtype), jax.ShapeDtypeStruct((ws_bytes,), jnp.uint8)),
    )
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
