"""ctypes binding of ``librpa_mi355x.so`` (declared in ``include/rpa_mi355x.h``).

There is no fallback: if the shared library is missing or does not load, importing the
op fails with an error that says how to build it.
"""

from __future__ import annotations

import ctypes
import os
from pathlib import Path

# RPA_LIBRARY points at another build of the same library (e.g. one compiled with different tile constants).
LIB_PATH = Path(os.environ.get("RPA_LIBRARY") or Path(__file__).resolve().parent / "lib" / "librpa_mi355x.so")

RPA_ABI_VERSION = 6
RPA_DTYPE_BF16, RPA_DTYPE_F32, RPA_DTYPE_FP8_E4M3, RPA_DTYPE_FP8_E5M2 = 0, 1, 2, 3
RPA_COMPUTE_BF16, RPA_COMPUTE_F32 = 0, 1
RPA_FLAG_FORCE_GENERIC = 1
RPA_FLAG_FP32_LOGITS = 2
RPA_FLAG_PREFILL_TILES = 4
RPA_FLAG_PIPE_TILES = 8
RPA_FLAG_PLAIN_TILES = 16
RPA_FLAG_NO_LOGIT_STASH = 32

EXPORTED_SYMBOLS = (
    "rpa_abi_version",
    "rpa_last_error",
    "rpa_workspace_bytes",
    "rpa_kernel_path",
    "rpa_workspace_init",
    "rpa_fwd_launch",
    "rpa_fwd_launch_static",
    "rpa_static_scratch_bytes",
    "rpa_v3_launch",
    "rpa_v3_workspace_bytes",
    "rpa_page_attention_workspace_bytes",
    "rpa_page_attention_launch",
    "rpa_ragged_decode_workspace_bytes",
    "rpa_ragged_decode_launch",
)


class RpaParams(ctypes.Structure):
    """Field-for-field image of ``struct RpaParams``."""

    _fields_ = [
        ("queries", ctypes.c_void_p),
        ("kv_pages", ctypes.c_void_p),
        ("context_lens", ctypes.c_void_p),
        ("block_tables", ctypes.c_void_p),
        ("query_start_loc", ctypes.c_void_p),
        ("num_seqs", ctypes.c_void_p),
        ("sinks", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_uint64),
        ("total_tokens", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("page_size", ctypes.c_int32),
        ("num_pages", ctypes.c_int32),
        ("max_num_seqs", ctypes.c_int32),
        ("pages_per_seq", ctypes.c_int32),
        ("num_sinks", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("logits_soft_cap", ctypes.c_float),
        ("sliding_window", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("compute", ctypes.c_int32),
        ("num_queries_per_block", ctypes.c_int32),
        ("num_kv_pages_per_block", ctypes.c_int32),
        ("num_warps", ctypes.c_int32),
        ("num_stages", ctypes.c_int32),
        ("flags", ctypes.c_uint32),
        ("q_scale", ctypes.c_float),
        ("k_scale", ctypes.c_float),
        ("v_scale", ctypes.c_float),
        ("kv_start", ctypes.c_void_p),
    ]


class RpaV3Params(ctypes.Structure):
    """Field-for-field image of ``struct RpaV3Params``."""

    _fields_ = [
        ("attn", RpaParams),
        ("new_keys", ctypes.c_void_p),
        ("new_values", ctypes.c_void_p),
        ("cache_dtype", ctypes.c_int32),
        ("cache_head_dim", ctypes.c_int32),
        ("cache_combined_heads", ctypes.c_int32),
        ("reserved", ctypes.c_int32),
    ]


class RpaPageAttnParams(ctypes.Structure):
    """Field-for-field image of ``struct RpaPageAttnParams``."""

    _fields_ = [
        ("query", ctypes.c_void_p),
        ("key_cache", ctypes.c_void_p),
        ("value_cache", ctypes.c_void_p),
        ("context_lens", ctypes.c_void_p),
        ("block_tables", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_uint64),
        ("num_seqs", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("block_size", ctypes.c_int32),
        ("num_blocks", ctypes.c_int32),
        ("max_blocks", ctypes.c_int32),
        ("attn_scale", ctypes.c_float),
        ("dtype", ctypes.c_int32),
        ("compute", ctypes.c_int32),
        ("flags", ctypes.c_uint32),
    ]


class RpaRaggedDecodeParams(ctypes.Structure):
    """Field-for-field image of ``struct RpaRaggedDecodeParams``."""

    _fields_ = [
        ("query", ctypes.c_void_p),
        ("key", ctypes.c_void_p),
        ("value", ctypes.c_void_p),
        ("sequence_start", ctypes.c_void_p),
        ("sequence_end", ctypes.c_void_p),
        ("out", ctypes.c_void_p),
        ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_uint64),
        ("batch", ctypes.c_int32),
        ("num_q_heads", ctypes.c_int32),
        ("num_kv_heads", ctypes.c_int32),
        ("head_dim", ctypes.c_int32),
        ("seq_len", ctypes.c_int32),
        ("softmax_scale", ctypes.c_float),
        ("logits_soft_cap", ctypes.c_float),
        ("window_left", ctypes.c_int32),
        ("dtype", ctypes.c_int32),
        ("compute", ctypes.c_int32),
        ("flags", ctypes.c_uint32),
        ("softmax_aux", ctypes.c_void_p),
        ("num_sinks", ctypes.c_int32),
        ("aux_rows", ctypes.c_int32),
    ]


RPA_MAX_SINK_KEYS = 64


class NativeLibraryError(RuntimeError):
    pass


_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise NativeLibraryError(
            f"{LIB_PATH} is missing: build it with `python -m ejkernel_amd.build` "
            "(hipcc, --offload-arch=gfx950). There is no CPU or eager fallback."
        )
    try:
        lib = ctypes.CDLL(str(LIB_PATH))
    except OSError as e:  # pragma: no cover - depends on the host
        raise NativeLibraryError(f"cannot load {LIB_PATH}: {e}") from e
    for name in EXPORTED_SYMBOLS:
        if not hasattr(lib, name):
            raise NativeLibraryError(f"{LIB_PATH} does not export {name}")
    lib.rpa_abi_version.restype = ctypes.c_int
    lib.rpa_abi_version.argtypes = []
    lib.rpa_last_error.restype = ctypes.c_char_p
    lib.rpa_last_error.argtypes = []
    lib.rpa_workspace_bytes.restype = ctypes.c_uint64
    lib.rpa_workspace_bytes.argtypes = [ctypes.POINTER(RpaParams)]
    lib.rpa_kernel_path.restype = ctypes.c_int
    lib.rpa_kernel_path.argtypes = [ctypes.POINTER(RpaParams)]
    lib.rpa_workspace_init.restype = ctypes.c_int
    lib.rpa_workspace_init.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p]
    lib.rpa_fwd_launch.restype = ctypes.c_int
    lib.rpa_fwd_launch.argtypes = [ctypes.POINTER(RpaParams), ctypes.c_void_p]
    lib.rpa_fwd_launch_static.restype = ctypes.c_int
    lib.rpa_fwd_launch_static.argtypes = [ctypes.POINTER(RpaParams), ctypes.c_void_p]
    lib.rpa_static_scratch_bytes.restype = ctypes.c_uint64
    lib.rpa_static_scratch_bytes.argtypes = []
    lib.rpa_v3_workspace_bytes.restype = ctypes.c_uint64
    lib.rpa_v3_workspace_bytes.argtypes = [ctypes.POINTER(RpaV3Params)]
    lib.rpa_v3_launch.restype = ctypes.c_int
    lib.rpa_v3_launch.argtypes = [ctypes.POINTER(RpaV3Params), ctypes.c_void_p]
    lib.rpa_page_attention_workspace_bytes.restype = ctypes.c_uint64
    lib.rpa_page_attention_workspace_bytes.argtypes = [ctypes.POINTER(RpaPageAttnParams)]
    lib.rpa_page_attention_launch.restype = ctypes.c_int
    lib.rpa_page_attention_launch.argtypes = [ctypes.POINTER(RpaPageAttnParams), ctypes.c_void_p]
    lib.rpa_ragged_decode_workspace_bytes.restype = ctypes.c_uint64
    lib.rpa_ragged_decode_workspace_bytes.argtypes = [ctypes.POINTER(RpaRaggedDecodeParams)]
    lib.rpa_ragged_decode_launch.restype = ctypes.c_int
    lib.rpa_ragged_decode_launch.argtypes = [ctypes.POINTER(RpaRaggedDecodeParams), ctypes.c_void_p]
    if lib.rpa_abi_version() != RPA_ABI_VERSION:
        raise NativeLibraryError(
            f"{LIB_PATH} has ABI version {lib.rpa_abi_version()}, this package expects {RPA_ABI_VERSION}: rebuild it"
        )
    _lib = lib
    return lib


def last_error() -> str:
    return load().rpa_last_error().decode("utf-8", "replace")
