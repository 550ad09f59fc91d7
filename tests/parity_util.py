"""Helpers shared by the GPU parity tests: the reference-generated codebook tables and the
output bound of the path."""

from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np

_GOLDEN = Path(__file__).resolve().parent / "golden" / "codebooks_v2.json"
_tables: dict | None = None


def reference_tables(dim: int, bits: int):
    """(centroids, boundaries) as fp32 arrays: the table the reference's own generator wrote for
    (dim, bits) when tests/golden/make_codebook_golden.py ran it (every configuration dimension at
    2/3/4/6/8 bits), else the oracle's scipy-based table (equal within one ulp where both exist)."""
    global _tables
    if _tables is None:
        _tables = json.loads(_GOLDEN.read_text())["tables"]
    entry = _tables.get(f"dim{dim}_bits{bits}")
    if entry is None:
        from oracle import oracle_np

        return oracle_np.lloyd_max_tables(dim, bits)
    cents = np.array(entry["centroids_u32"], dtype=np.int32).view(np.float32)
    bounds = np.array(entry["boundaries_u32"], dtype=np.int32).view(np.float32)
    return cents.copy(), bounds.copy()


def output_error(got, want, s, r, k, out_is_16bit: bool, out_is_bf16: bool = True):
    """Worst error of `got` against the fp64 reference `want` as a fraction of the path's bound
    2e-2 * ||x|| * ||w_row|| / sqrt(K), two ways: `strict` against the bound alone, and `rounded`
    with the half-ulp the 16-bit output format itself may add to any result (2^-8 relative for
    bf16, 2^-11 for fp16) added to the bound.  fp32 outputs: both are the same number."""
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    bound = 2e-2 * np.asarray(s, np.float64)[:, None] * np.asarray(r, np.float64)[None, :] / math.sqrt(k)
    err = np.abs(got - want)
    strict = float((err / (bound + 1e-300)).max())
    if not out_is_16bit:
        return strict, strict
    half_ulp = 2.0 ** -8 if out_is_bf16 else 2.0 ** -11
    rounded = float((err / (bound + np.abs(want) * half_ulp + 1e-300)).max())
    return strict, rounded


def outside_rounded_bound(got, want, s, r, k, out_is_bf16: bool = True) -> int:
    """For a 16-bit output: the number of elements that are NOT the rounding of any value within the stated
    bound of `want`.  Rounding to the output format is monotonic, so that is
        round(want - bound) <= got <= round(want + bound)
    element by element.  Zero means: wherever a stored output exceeds the bound, the excess is the rounding
    of the stored 16-bit value and nothing else - the kernel's result before that rounding may have met it."""
    import torch

    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    bound = 2e-2 * np.asarray(s, np.float64)[:, None] * np.asarray(r, np.float64)[None, :] / math.sqrt(k)
    dtype = torch.bfloat16 if out_is_bf16 else torch.float16

    def rounded(a):
        return torch.from_numpy(a).to(torch.float32).to(dtype).double().numpy()
    # (the fp64 -> fp32 step before the 16-bit rounding is widened by one fp32 spacing: it must not tighten the interval)
    lo = rounded(np.nextafter((want - bound).astype(np.float32), np.float32(-np.inf)).astype(np.float64))
    hi = rounded(np.nextafter((want + bound).astype(np.float32), np.float32(np.inf)).astype(np.float64))
    return int(((got < lo) | (got > hi)).sum())


def cosine(got, want) -> float:
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return float((got * want).sum() / (np.linalg.norm(got) * np.linalg.norm(want) + 1e-300))
