"""Compile ``libtwilight_hip.so`` for gfx950 with hipcc (no GPU needed: it cross-compiles)."""
from __future__ import annotations

import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

_PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_PKG, "csrc")
LIB_PATH = os.path.join(_PKG, "libtwilight_hip.so")
SOURCES = ["api.hip", "top_p.hip", "top_p_dtype.hip", "gemv_int4.hip", "fused_row.hip", "layer_row.hip", "gemv_nhd.hip", "sparse_attn.hip", "group_attn.hip", "rope.hip", "quest.hip", "kv_shadow.hip", "meta_planes.hip", "label_ops.hip", "qk_int8.hip"]

# Packed-fp32 VALU forms are disabled for every kernel of this library.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: libtwilight_hip.so cannot be built")
    return exe


def build_library(verbose: bool = False, jobs: int = 6) -> str:
    """Compile every source of ``csrc/`` and link the shared library in-tree. Always recompiles."""
    hipcc = _hipcc()
    objdir = os.path.join(_PKG, "build")
    os.makedirs(objdir, exist_ok=True)

    def compile_one(src: str) -> str:
        obj = os.path.join(objdir, src.replace(".hip", ".o"))
        cmd = [hipcc, *HIPCC_FLAGS, "-c", os.path.join(CSRC, src), "-o", obj]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{r.stdout}\n{r.stderr}")
        if verbose:
            # the host pass does not know the device-only feature flag; that warning is expected
            noise = [ln for ln in r.stderr.splitlines() if ln.strip() and "packed-fp32-ops" not in ln]
            if noise:
                print("\n".join(noise))
        return obj

    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(compile_one, SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", tmp]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError(f"link failed:\n{r.stdout}\n{r.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
