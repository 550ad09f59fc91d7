"""Build the C oracle (and, where the reference checkout is present, the
reference's own CPU matmul kernels) into shared libraries next to this file.

    python oracle/build.py            # oracle/liboq_oracle.so (+ oracle/_ref/...)
"""

from __future__ import annotations

import os
import subprocess
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
ORACLE_SO = HERE / "liboq_oracle.so"
REF_DIR = HERE / "_ref"
REF_SO = REF_DIR / "liboq_ref_cpu.so"
REFERENCE_ROOT = Path(os.environ.get("OQ_REFERENCE_ROOT", "/root/reference"))
REF_CPU = REFERENCE_ROOT / "native-kernels/orbitquant-packed-matmul/orbitquant_packed_matmul_cpu"


def build_oracle() -> Path:
    cmd = [
        "gcc", "-O3", "-march=x86-64-v3", "-ffp-contract=off", "-fopenmp", "-shared", "-fPIC",
        "-o", str(ORACLE_SO), str(HERE / "oq_oracle.c"), "-lm",
    ]
    subprocess.run(cmd, check=True)
    return ORACLE_SO


def build_reference_cpu() -> Path | None:
    """Compile the reference's scalar/AVX2/AVX-512 packed-matmul range kernels
    from where they lie, plus this repo's C-ABI shim around their C++ interface.
    Returns None when the reference checkout (or torch's header-only BFloat16/
    Half headers it includes) is not present."""
    shim = HERE / "ref_cpu_shim.cpp"
    if not REF_CPU.is_dir() or not shim.exists():
        return None
    try:
        import torch
    except Exception:
        return None
    include = Path(torch.__file__).resolve().parent / "include"
    if not (include / "torch/headeronly/util/BFloat16.h").exists():
        return None
    REF_DIR.mkdir(exist_ok=True)
    sources = [
        REF_CPU / "packed_matmul_scalar.cpp",
        REF_CPU / "packed_matmul_x86.cpp",
        REF_CPU / "packed_matmul_x86_avx512.cpp",
    ]
    cmd = [
        "g++", "-std=c++17", "-O3", "-fopenmp", "-shared", "-fPIC",
        f"-I{REF_CPU}", f"-I{include}", "-o", str(REF_SO), str(shim),
    ] + [str(s) for s in sources]
    subprocess.run(cmd, check=True)
    return REF_SO


def main() -> int:
    print("built", build_oracle())
    ref = build_reference_cpu()
    print("built", ref) if ref else print("reference CPU kernels: not built")
    return 0


if __name__ == "__main__":
    sys.exit(main())
