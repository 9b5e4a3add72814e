"""Compile the HIP sources into ``lib/libcosmosfp8.so`` for gfx950 (and nothing else).

``hipcc`` cross-compiles without a GPU.  The library is built in-tree so that it
travels with the source checkout; it is never installed into site-packages.
"""
from __future__ import annotations

import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
CSRC_DIR = PKG_DIR.parent / "csrc"
INCLUDE_DIR = PKG_DIR.parent.parent / "include"
LIB_DIR = PKG_DIR / "lib"
LIB_PATH = LIB_DIR / "libcosmosfp8.so"
OBJ_DIR = CSRC_DIR / "build"

SOURCES = ["api.hip", "quant_rowwise.hip", "quant_tensorwise.hip", "quant_block.hip", "gemm_fp8.hip", "gemm_grouped_xres.hip", "moe_indices.hip",
           "quant_mxfp4.hip", "gemm_mxfp4.hip"]

# Per-file flags.  gemm_grouped_xres.hip: matrix instructions write ordinary vector registers (see the file's header).
EXTRA_FLAGS = {"gemm_grouped_xres.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form"]}

# -packed-fp32-ops: hipcc must not form v_pk_{add,mul,fma}_f32 (they have returned
# wrong results on some machines).  -ffp-contract=off: the quantisers rely on
# explicit fma placement for a correctly rounded quotient.
HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-ffp-contract=off",
    "-fhip-fp32-correctly-rounded-divide-sqrt",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the FP8 library cannot be built")
    return exe


def _compile(src: str) -> Path:
    obj = OBJ_DIR / (src.replace(".hip", ".o"))
    cmd = [hipcc(), *HIPCC_FLAGS, *EXTRA_FLAGS.get(src, []), f"-I{INCLUDE_DIR}", f"-I{CSRC_DIR}", "-c", str(CSRC_DIR / src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stdout}\n{res.stderr}")
    return obj


def build(verbose: bool = False) -> Path:
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    LIB_DIR.mkdir(parents=True, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(_compile, SOURCES))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(tmp), *map(str, objs)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stdout}\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH}")
    return LIB_PATH


if __name__ == "__main__":
    build(verbose=True)
