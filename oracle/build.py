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
    checks = [
        "gcc", "-O2", "-march=x86-64-v3", "-ffp-contract=off", "-fopenmp", "-shared", "-fPIC",
        "-o", str(HERE / "liboq_kernel_checks.so"), str(HERE / "kernel_arith_check.c"), "-lm",
    ]
    subprocess.run(checks, check=True)
    return ORACLE_SO


def build_reference_cpu() -> Path | None:
    """Compile the reference's CPU kernels on this path (packed matmul + activation
    quantizer, with their thread pool and ISA dispatch) from where they lie, plus this
    repo's own operator registration (`ref_cpu_bind.cpp`), into oracle/_ref/.  The
    reference's generated binding glue is not used.  Returns None when the reference
    checkout is not present (e.g. on a GPU box, which only uses a prebuilt file)."""
    bind = HERE / "ref_cpu_bind.cpp"
    if not REF_CPU.is_dir():
        return None
    from torch.utils import cpp_extension

    import torch

    REF_DIR.mkdir(exist_ok=True)
    names = ["packed_matmul_cpu", "packed_matmul_scalar", "packed_matmul_x86", "packed_matmul_x86_avx512",
             "packed_matmul_neon", "quantize_activations_cpu", "cpu_pool", "cpu_threads", "cpu_isa"]
    sources = [REF_CPU / f"{n}.cpp" for n in names]
    includes = [f"-I{p}" for p in cpp_extension.include_paths()]
    lib_dir = Path(torch.__file__).resolve().parent / "lib"
    cmd = [
        "g++", "-std=c++17", "-O3", "-DCPU_KERNEL", "-shared", "-fPIC", "-pthread",
        f"-I{REF_CPU}", f"-I{REF_CPU.parent / 'torch-ext'}", *includes,
        "-o", str(REF_SO), str(bind), *[str(s) for s in sources],
        f"-L{lib_dir}", "-ltorch", "-ltorch_cpu", "-lc10", f"-Wl,-rpath,{lib_dir}",
    ]
    subprocess.run(cmd, check=True)
    return REF_SO


def main() -> int:
    print("built", build_oracle())
    ref = build_reference_cpu()
    print("built", ref) if ref else print("reference CPU kernels: not built")
    return 0


if __name__ == "__main__":
    sys.exit(main())
