"""Compile the gfx950 HIP kernels into `orbitquant_amd/liborbitquant_hip.so`.

    python -m orbitquant_amd.build

hipcc cross-compiles for gfx950 without a GPU.  The rotate+quantize kernel is
built without FMA contraction (its results must match the CPU statement of the
algorithm bit for bit); packed fp32 VALU instructions are disabled everywhere.

    python -m orbitquant_amd.build --variant stamps --flags=-DOQ_GEMM_STAMPS --only packed_gemm.hip

builds `liborbitquant_hip_stamps.so` beside the library: the listed sources compiled with the
extra flags, every other object taken from the last full build.  `ORBITQUANT_HIP_LIB=<path>`
makes the package load it.  (-DOQ_GEMM_STAMPS: the tile GEMM records the clock at its phase
boundaries, see `bench.py --gemm-phases`.)
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
# kernels whose leading scalar arguments are to arrive in scalar registers (see packed_gemm_kernel.h)
PRELOAD = ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
SOURCES = {
    "capi.hip": [],
    "rotate_quantize.hip": ["-ffp-contract=off"],
    "rotate_quantize_fast.hip": ["-ffp-contract=off"],
    "packed_generic.hip": [],
    "adaln_int4.hip": [],
    "pack_utils.hip": [],
    "packed_gemm.hip": PRELOAD,
    "packed_gemm_bytes.hip": PRELOAD,
    "packed_gemm_tiled.hip": PRELOAD,
    "packed_gemm_staged.hip": PRELOAD,
    "packed_gemm_splitk.hip": [],
    "packed_gemm_av.hip": [],
    "packed_gemv.hip": PRELOAD,
    "packed_gemv_group.hip": [],
    "packed_gemv_rows.hip": [],
    "token_linear.hip": [],
    "token_linear_w2.hip": [],
    "token_linear_w3.hip": [],
    "token_linear_w4.hip": [],
}


INCREMENTAL = False


def _compile(item, obj_dir: Path = None) -> Path:
    name, extra = item
    obj = (obj_dir or OBJ_DIR) / (name + ".o")
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


def build_variant(variant: str, flags: list, only: list) -> Path:
    """The library with `only` recompiled under `flags`; the other objects come from the full build."""
    obj_dir = PKG / f"build_{variant}"
    obj_dir.mkdir(exist_ok=True)
    missing = [n for n in SOURCES if n not in only and not (OBJ_DIR / (n + ".o")).exists()]
    if missing:
        raise SystemExit(f"run the full build first: no object for {missing}")
    with ThreadPoolExecutor(max_workers=4) as pool:
        changed = dict(zip(only, pool.map(lambda n: _compile((n, SOURCES[n] + flags), obj_dir), only)))
    objects = [str(changed.get(n, OBJ_DIR / (n + ".o"))) for n in SOURCES]
    lib = PKG / f"liborbitquant_hip_{variant}.so"
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(lib)] + objects, check=True)
    print("built", lib)
    return lib


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser()
    ap.add_argument("--incremental", action="store_true")
    ap.add_argument("--variant", default=None)
    ap.add_argument("--flags", default="")
    ap.add_argument("--only", default="")
    opts = ap.parse_args()
    INCREMENTAL = opts.incremental
    if opts.variant:
        build_variant(opts.variant, opts.flags.split(), [n for n in opts.only.split(",") if n])
    else:
        build()
    sys.exit(0)
