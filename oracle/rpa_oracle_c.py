"""ctypes wrapper of the C restatement (``rpa_oracle.c``).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

from .rpa_oracle import _sinks_per_q_head, bf16_bits, bf16_from_bits

_DIR = Path(__file__).resolve().parent
LIB_PATH = _DIR / "_build" / "librpa_oracle.so"
_lib = None


def build() -> Path:
    subprocess.run(["make", "-C", str(_DIR)], check=True, capture_output=True)
    return LIB_PATH


def load():
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        lib = ctypes.CDLL(str(LIB_PATH))
        lib.rpa_oracle_strict.restype = ctypes.c_int
        lib.rpa_oracle_strict.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int] * 8 + [
            ctypes.c_float, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
            ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        lib.rpa_oracle_max_threads.restype = ctypes.c_int
        _lib = lib
    return _lib


def max_threads() -> int:
    return int(load().rpa_oracle_max_threads())


def rpa_strict_c(queries, kv_pages, context_lens, block_tables, query_start_loc, num_seqs, softmax_scale=None,
                 logits_soft_cap=None, sliding_window=None, softmax_aux=None, io_dtype="bfloat16", threads=0,
                 aux_dtype="float32"):
    """Same contract as ``rpa_oracle.rpa_strict`` (compute dtype == io dtype): float32 arrays holding
    ``io_dtype``-representable values in, float32 ``[T, Hq, D]`` out."""
    lib = load()
    bf = io_dtype in ("bfloat16", "bf16")
    q = np.ascontiguousarray(queries, np.float32)
    kv = np.ascontiguousarray(kv_pages, np.float32)
    T, Hq, D = q.shape
    P, page, H2, _ = kv.shape
    Hkv = H2 // 2
    if bf:
        q_buf, kv_buf = bf16_bits(q), bf16_bits(kv)
        out = np.zeros((T, Hq, D), np.uint16)
    else:
        q_buf, kv_buf = q, kv
        out = np.zeros((T, Hq, D), np.float32)
    ctx = np.ascontiguousarray(context_lens, np.int32)
    bt = np.ascontiguousarray(block_tables, np.int32)
    cu = np.ascontiguousarray(query_start_loc, np.int32)
    n = int(np.asarray(num_seqs).reshape(-1)[0])
    sinks, n_sinks = None, 0
    if softmax_aux is not None:
        sinks = np.ascontiguousarray(_sinks_per_q_head(np.asarray(softmax_aux, np.float32), Hq, Hkv), np.float32)
        n_sinks = sinks.shape[1]
    scale = D**-0.5 if softmax_scale is None else float(softmax_scale)
    rc = lib.rpa_oracle_strict(
        q_buf.ctypes.data, kv_buf.ctypes.data, ctx.ctypes.data, bt.ctypes.data, cu.ctypes.data, n, T, Hq, Hkv, D, page, P,
        bt.shape[-1], scale, 0.0 if logits_soft_cap is None else float(logits_soft_cap),
        0 if sliding_window is None else int(sliding_window), None if sinks is None else sinks.ctypes.data, n_sinks,
        1 if bf else 0, out.ctypes.data, int(threads), 1 if aux_dtype in ("bfloat16", "bf16") else 0)
    if rc != 0:
        raise RuntimeError("rpa_oracle_strict failed")
    return bf16_from_bits(out) if bf else out
