"""CPU checks of two arithmetic shortcuts of the plan-based rotate+quantize kernel, on models of
them in C (oracle/kernel_arith_check.c) against the plain IEEE operations: the four-instruction
division, over billions of operand pairs of the admitted ranges, and the folding of the
1/sqrt(block) factor into the bucketize thresholds, around every boundary of the codebooks."""

from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent


@pytest.fixture(scope="module")
def checks():
    so = ROOT / "oracle" / "liboq_kernel_checks.so"
    if not so.exists():
        from oracle.build import build_oracle

        build_oracle()
    lib = ctypes.CDLL(str(so))
    f32p = ctypes.POINTER(ctypes.c_float)
    lib.oqk_division_mismatches.restype = ctypes.c_int64
    lib.oqk_division_mismatches.argtypes = [ctypes.c_int64, ctypes.c_uint64, ctypes.c_int, f32p, f32p]
    lib.oqk_fold_threshold.restype = ctypes.c_float
    lib.oqk_fold_threshold.argtypes = [ctypes.c_float, ctypes.c_float]
    lib.oqk_fold_mismatches.restype = ctypes.c_int64
    lib.oqk_fold_mismatches.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_int]
    return lib


@pytest.mark.parametrize("mode", [0, 1, 2])
def test_four_instruction_division_is_the_ieee_quotient(checks, mode):
    x, d = ctypes.c_float(), ctypes.c_float()
    bad = checks.oqk_division_mismatches(1_000_000_000, 11 + mode, mode, ctypes.byref(x), ctypes.byref(d))
    assert bad == 0, f"{bad} quotients differ, first x={x.value!r} d={d.value!r}"


def test_the_division_check_catches_an_inexact_sequence(checks):
    x, d = ctypes.c_float(), ctypes.c_float()
    assert checks.oqk_division_mismatches(200_000_000, 5, 16, ctypes.byref(x), ctypes.byref(d)) > 0


@pytest.mark.parametrize("block", [8, 64, 128, 512, 2048, 4096])
def test_folded_thresholds_decide_like_multiply_then_compare(checks, block):
    from oracle import oracle_np

    c = np.float32(1.0 / np.sqrt(block))
    for bits in (2, 3, 4, 6):
        _, bounds = oracle_np.lloyd_max_tables(max(block, 64), bits)
        for b in bounds:
            assert checks.oqk_fold_mismatches(float(b), float(c), 4096) == 0
    # boundaries no codebook has: zero, denormals, huge, infinities
    for b in (0.0, -0.0, 1e-45, -1e-45, 1e-38, 3e38, -3e38, float("inf"), float("-inf")):
        assert checks.oqk_fold_mismatches(b, float(c), 4096) == 0
    t = checks.oqk_fold_threshold(float("nan"), float(c))
    assert t != t
