"""Build libtybok_hip.so for gfx950 with plain hipcc (no torch headers, no pybind).

Run as ``python -m tybok_amd.csrc.build`` or through ``__graft_entry__.build()``.  hipcc
cross-compiles without a GPU; the library lands in ``tybok_amd/_lib/`` next to the package so it
travels with the source tree.
"""

from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(os.path.dirname(HERE), "_lib")
LIB_PATH = os.path.join(LIB_DIR, "libtybok_hip.so")
SOURCES = ("fp8w_gemm.hip", "fp8w_gemm_wide.hip", "expert_attn.hip", "expert_attn_d256.hip", "expert_attn_px.hip", "expert_tail.hip", "expert_kv_proj.hip", "layer_norm.hip", "tower_attn.hip", "rope_rows.hip", "tk_api.hip")
ARCH = "gfx950"


def hipcc_path() -> str:
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


def build_library(verbose: bool = True) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [
        hipcc_path(),
        f"--offload-arch={ARCH}",
        "-O3",
        "-std=c++17",
        "-fPIC",
        "-shared",
        # keep hipcc from forming packed-fp32 VALU ops out of ordinary float code
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        *[os.path.join(HERE, s) for s in SOURCES],
        "-o", LIB_PATH + ".tmp",
    ]  # fmt: skip
    if verbose:
        print("[tybok_amd] " + " ".join(cmd), flush=True)
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(line for line in proc.stderr.splitlines() if noise not in line)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if err.strip() and verbose:
        print(err, file=sys.stderr)
    os.replace(LIB_PATH + ".tmp", LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library())
