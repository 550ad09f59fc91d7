"""Writes tests/golden/codebooks_v2.json: the fp32 Lloyd-Max tables of the
reference's v2 generator for the dimensions and bit widths of the benchmark
configurations, as raw uint32 bit patterns.

Run once, in the build container only (it loads the reference's
codebooks/lloyd_max.py from the read-only reference checkout; nothing of the
reference is copied).  The exact fp32 bits at these dimensions are not held by
any of the reference's own tests (they hold dim=32/bits=3 to 1e-6 only), which
is why this fixture exists.

    ORBITQUANT_DISABLE_CODEBOOK_DISK_CACHE=1 python tests/golden/make_codebook_golden.py
"""

from __future__ import annotations

import importlib.util
import json
import os
import sys
from pathlib import Path

REFERENCE = Path(os.environ.get("OQ_REFERENCE_ROOT", "/root/reference"))
DIMS = (24, 32, 64, 128, 512, 768, 1152, 1536, 3072, 4096, 4608, 5120, 12288, 13824, 14336)
BITS = (2, 3, 4, 6)


def main() -> int:
    os.environ["ORBITQUANT_DISABLE_CODEBOOK_DISK_CACHE"] = "1"
    path = REFERENCE / "src/orbitquant/codebooks/lloyd_max.py"
    spec = importlib.util.spec_from_file_location("_ref_lloyd_max", path)
    module = importlib.util.module_from_spec(spec)
    sys.modules["_ref_lloyd_max"] = module
    spec.loader.exec_module(module)
    tables = {}
    for dim in DIMS:
        for bits in BITS:
            book = module._generate_exact_v2_codebook(dim, bits)
            tables[f"dim{dim}_bits{bits}"] = {
                "centroids_u32": book.centroids.view(dtype=__import__("torch").int32).tolist(),
                "boundaries_u32": book.boundaries.view(dtype=__import__("torch").int32).tolist(),
            }
    out = Path(__file__).resolve().parent / "codebooks_v2.json"
    out.write_text(json.dumps({"algorithm_version": 2, "tables": tables}, indent=0))
    print("wrote", out, len(tables), "tables")
    return 0


if __name__ == "__main__":
    sys.exit(main())
