"""Build libtybok_hip.so for gfx950 with plain hipcc (no torch headers, no pybind).

Run as ``python -m tybok_amd.csrc.build`` or through ``__graft_entry__.build()``.  hipcc
cross-compiles without a GPU; the library lands in ``tybok_amd/_lib/`` next to the package so it
travels with the source tree.  Each translation unit is compiled to an object of its own (in
parallel) and the objects are linked into the shared library.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(os.path.dirname(HERE), "_lib")
OBJ_DIR = os.path.join(LIB_DIR, "obj")
LIB_PATH = os.path.join(LIB_DIR, "libtybok_hip.so")
SOURCES = ("fp8w_gemm.hip", "fp8w_gemm_stream.hip", "fp8w_gemm_wide.hip", "expert_attn.hip", "expert_attn_d256.hip", "expert_attn_px.hip", "expert_tail.hip", "expert_kv_proj.hip", "layer_norm.hip", "tower_attn.hip", "rope_rows.hip", "prefix_prep.hip", "stream_read.hip", "w8a8_gemm.hip", "bf16w_gemm_wide.hip", "tk_api.hip")
HEADERS = ("tk_common.h", "tk_kernels.h", os.path.join("..", "..", "include", "tybok_hip.h"))
ARCH = "gfx950"
FLAGS = (
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    # keep hipcc from forming packed-fp32 VALU ops out of ordinary float code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)  # fmt: skip
_NOISE = "is not a recognized feature for this target"


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


def _run(cmd: list[str], verbose: bool) -> None:
    if verbose:
        print("[tybok_amd] " + " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(line for line in proc.stderr.splitlines() if _NOISE not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}): {' '.join(cmd)}\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)


def build_library(verbose: bool = True, incremental: bool = False, jobs: int = 8) -> str:
    """Compile every source and link the library.  ``incremental`` skips objects that are newer than
    their source and the shared headers (development convenience; the default compiles everything)."""
    os.makedirs(OBJ_DIR, exist_ok=True)
    hipcc = hipcc_path()
    newest_header = max(os.path.getmtime(os.path.join(HERE, h)) for h in HEADERS)
    todo, objects = [], []
    for s in SOURCES:
        src = os.path.join(HERE, s)
        obj = os.path.join(OBJ_DIR, s.replace(".hip", ".o"))
        objects.append(obj)
        if incremental and os.path.exists(obj) and os.path.getmtime(obj) >= max(os.path.getmtime(src), newest_header):
            continue
        todo.append([hipcc, *FLAGS, "-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=max(1, min(jobs, len(todo) or 1))) as pool:
        list(pool.map(lambda cmd: _run(cmd, verbose), todo))
    _run([hipcc, f"--offload-arch={ARCH}", "-shared", "-fPIC", *objects, "-o", LIB_PATH + ".tmp"], verbose)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(incremental="--incremental" in sys.argv))
