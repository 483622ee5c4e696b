"""Builds libdg_attn_hip.so (gfx950) in-tree with hipcc.

hipcc cross-compiles without a GPU.  Flags: packed-FP32 instruction selection is switched
off for every HIP translation unit (hipcc then emits scalar v_mul/v_fma for float math).
"""
from __future__ import annotations

import os
import shutil
import subprocess
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC = PKG_DIR / "csrc"
LIB_NAME = "libdg_attn_hip.so"
LIB_PATH = PKG_DIR / LIB_NAME
SOURCES = ["dg_attn_api.hip", "attn_mfma.hip", "attn_wsplit.hip", "attn_aux.hip", "qk_rope_kv.hip", "attn_topk.hip", "kv_snapshot.hip"]
HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc_path() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


def build_library(verbose: bool = False) -> Path:
    """Compile every HIP source and link the shared library next to this package."""
    hipcc = hipcc_path()
    obj_dir = PKG_DIR / "build"
    obj_dir.mkdir(exist_ok=True)
    objs = []
    procs = []
    for src in SOURCES:
        obj = obj_dir / (Path(src).stem + ".o")
        cmd = [hipcc, *HIP_FLAGS, "-c", str(CSRC / src), "-o", str(obj)]
        if verbose:
            print(" ".join(cmd), flush=True)
        procs.append((src, subprocess.Popen(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)))
        objs.append(str(obj))
    for src, proc in procs:
        out, _ = proc.communicate()
        if proc.returncode != 0:
            raise RuntimeError(f"hipcc failed on {src}:\n{out}")
    tmp = PKG_DIR / (LIB_NAME + ".tmp")
    cmd = [hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", *objs, "-o", str(tmp)]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
