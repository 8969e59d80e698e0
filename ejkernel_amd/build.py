"""Builds ``librpa_mi355x.so`` (HIP kernels + C ABI) for gfx950 with hipcc.

``python -m ejkernel_amd.build`` compiles every source under ``csrc/`` in-tree; the
resulting shared object sits next to this file under ``lib/`` and is what
``ejkernel_amd._native`` loads.  hipcc cross-compiles, so no GPU is needed to build.
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "librpa_mi355x.so"
OBJ_DIR = PKG_DIR / "build"

SOURCES = ["rpa_api.hip", "rpa_generic.hip", "rpa_kv_update.hip", "rpa_sink_keys.hip", "rpa_tile.hip"]
# -packed-fp32-ops is switched off on purpose: the compiler must not form v_pk_*_f32.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
    "-Wno-unknown-warning-option",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; librpa_mi355x.so cannot be built")
    return exe


def _compile(src: str, extra: list[str]) -> Path:
    obj = OBJ_DIR / (Path(src).stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{r.stdout}\n{r.stderr}")
    # the host pass warns that it does not know the packed-fp32 feature: harmless
    return obj


def build(verbose: bool = True, extra_flags: list[str] | None = None, jobs: int = 4) -> Path:
    """Compile all sources and link the shared library. Always recompiles."""
    extra = list(extra_flags or [])
    OBJ_DIR.mkdir(exist_ok=True)
    LIB_DIR.mkdir(exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, extra), SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({LIB_PATH.stat().st_size} bytes)")
    return LIB_PATH


if __name__ == "__main__":
    build(extra_flags=sys.argv[1:])
