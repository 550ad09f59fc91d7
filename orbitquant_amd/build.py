"""Compile the gfx950 HIP kernels into `orbitquant_amd/liborbitquant_hip.so`.

    python -m orbitquant_amd.build

hipcc cross-compiles for gfx950 without a GPU.  The rotate+quantize kernel is
built without FMA contraction (its results must match the CPU statement of the
algorithm bit for bit); packed fp32 VALU instructions are disabled everywhere.
"""

from __future__ import annotations

import os
import subprocess
import sys
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB = PKG / "liborbitquant_hip.so"
OBJ_DIR = PKG / "build"

COMMON = [
    "hipcc", "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fno-gpu-flush-denormals-to-zero", "-Wno-unused-command-line-argument",
]
SOURCES = {
    "capi.hip": [],
    "rotate_quantize.hip": ["-ffp-contract=off"],
    "rotate_quantize_fast.hip": ["-ffp-contract=off"],
    "packed_generic.hip": [],
    "adaln_int4.hip": [],
    "pack_utils.hip": [],
    "packed_gemm.hip": [],
    "packed_gemm_bytes.hip": [],
    "packed_gemm_tiled.hip": [],
    "packed_gemm_staged.hip": [],
    "packed_gemm_splitk.hip": [],
    "packed_gemm_av.hip": [],
    "packed_gemv.hip": [],
    "packed_gemv_group.hip": [],
    "packed_gemv_rows.hip": [],
    "token_linear.hip": [],
    "token_linear_w2.hip": [],
    "token_linear_w3.hip": [],
    "token_linear_w4.hip": [],
}


INCREMENTAL = False


def _compile(item) -> Path:
    name, extra = item
    obj = OBJ_DIR / (name + ".o")
    if INCREMENTAL and obj.exists():
        newest = max(p.stat().st_mtime for p in list(CSRC.glob("*.h")) + [CSRC / name, PKG.parent / "include/orbitquant_hip.h"])
        if obj.stat().st_mtime > newest:
            return obj
    cmd = COMMON + extra + os.environ.get("OQ_HIPCC_FLAGS", "").split() + ["-c", str(CSRC / name), "-o", str(obj)]
    t0 = time.time()
    proc = subprocess.run(cmd, stderr=subprocess.PIPE, text=True)
    noise = "'-packed-fp32-ops' is not a recognized feature for this target"  # host pass only
    for line in proc.stderr.splitlines():
        if noise not in line:
            print(line, file=sys.stderr)
    if proc.returncode != 0:
        raise subprocess.CalledProcessError(proc.returncode, cmd)
    print(f"  compiled {name} in {time.time() - t0:.1f}s", flush=True)
    return obj


def build(verbose: bool = True) -> Path:
    OBJ_DIR.mkdir(exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as pool:
        objects = list(pool.map(_compile, SOURCES.items()))
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB)] + [str(o) for o in objects]
    subprocess.run(cmd, check=True)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    INCREMENTAL = "--incremental" in sys.argv
    build()
    sys.exit(0)
