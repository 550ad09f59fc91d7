"""Writes tests/golden/rotations.json: SHA-256 and the first 16 entries of the
RPBH permutation / sign draws for the benchmark dimensions.  Uses plain torch
only (torch.Generator + randperm + randint, the calls the reference's
rotations/rpbh.py:55-65 makes); it guards against a torch build whose CPU
generator stream differs from the one the fixtures were made with.

    python tests/golden/make_rotation_golden.py
"""

from __future__ import annotations

import hashlib
import json
from pathlib import Path

import torch

CASES = [(8, 5), (24, 17), (24, 29), (1152, 0), (3072, 0), (4096, 0), (4608, 0), (5120, 0),
         (12288, 0), (13824, 0), (14336, 0)]


def draw(dim: int, seed: int):
    gen = torch.Generator(device="cpu")
    gen.manual_seed(seed)
    perm = torch.randperm(dim, generator=gen, dtype=torch.long, device="cpu")
    signs = torch.randint(0, 2, (dim,), generator=gen, dtype=torch.int8, device="cpu") * 2 - 1
    return perm, signs


def main() -> None:
    out = {}
    for dim, seed in CASES:
        perm, signs = draw(dim, seed)
        out[f"dim{dim}_seed{seed}"] = {
            "perm_sha256": hashlib.sha256(perm.numpy().astype("<i8").tobytes()).hexdigest(),
            "signs_sha256": hashlib.sha256(signs.numpy().astype("i1").tobytes()).hexdigest(),
            "perm_head": perm[:16].tolist(),
            "signs_head": signs[:16].tolist(),
        }
    path = Path(__file__).resolve().parent / "rotations.json"
    path.write_text(json.dumps({"torch": torch.__version__, "draws": out}, indent=1))
    print("wrote", path)


if __name__ == "__main__":
    main()
