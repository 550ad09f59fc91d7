"""The oracle fixes the summation order of the token norm (the reference's `torch.norm` order is
implementation-defined and differs between its own back-ends), so its codes can differ from the
Python specification's where, and only where, the last bit of a norm moves a rotated value
across a boundary it sits on.  This test restates the specification with plain torch operations
(src/orbitquant/functional.py:16-22: `norm`, `/`; src/orbitquant/rotations/rpbh.py:74-84:
`index_select`, `*`, the reshape/cat butterflies of src/orbitquant/rotations/fwht.py:19-25, the
multiply by 1/sqrt(block); src/orbitquant/codebooks/lloyd_max.py:40-42: `bucketize`) on every
configuration's input distribution, counts the codes that differ from the oracle's, and checks
each one in fp64: the token's two norms differ (each within a few ulps of the exact norm), the
codes are neighbours, and the rotated value lies no further from the boundary between them than
the norms' difference and the fp32 rounding of the rotation can move it."""

from __future__ import annotations

import math

import numpy as np
import pytest
import torch

from oracle import oracle_c, oracle_np as o
from parity_util import reference_tables

CONFIGS = [
    # name, K, block, a_bits, dtype, rows, input kind
    ("c1", 1152, 64, 4, torch.float32, 2048, "entry_outliers"),
    ("c2 fc1", 1152, "paper", 4, torch.bfloat16, 2048, "column_outliers"),
    ("c2 fc2", 4608, "paper", 4, torch.bfloat16, 1024, "column_outliers"),
    ("c3", 3072, "paper", 3, torch.bfloat16, 1024, "student_t"),
    ("c3 fc2", 12288, "paper", 3, torch.bfloat16, 384, "student_t"),
    ("c4 fc1", 5120, "paper", 6, torch.bfloat16, 768, "entry_outliers"),
    ("c4 fc2", 13824, "paper", 6, torch.bfloat16, 320, "entry_outliers"),
    ("c5", 4096, "paper", 4, torch.bfloat16, 1024, "plain"),
    ("c5 down", 14336, "paper", 4, torch.bfloat16, 320, "plain"),
]


def make_input(kind, m, k, dtype, gen):
    x = torch.randn(m, k, generator=gen)
    if kind == "entry_outliers":
        x = torch.where(torch.rand(m, k, generator=gen) < 0.01, x * 20, x)
    elif kind == "column_outliers":
        cols = torch.randperm(k, generator=gen)[: max(1, math.ceil(0.005 * k))]
        x[:, cols] *= 30
    elif kind == "student_t":
        x = x / torch.sqrt(torch.randn(m, k, 4, generator=gen).square().sum(-1) / 4)
    return x.to(dtype)


def spec_codes(x, perm, signs, boundaries, block, eps):
    """The specification, operation by operation, in torch fp32 on the CPU."""
    work = x.to(torch.float32)
    norms = work.norm(dim=-1, keepdim=True)
    unit = work / (norms + eps)
    y = unit.index_select(dim=-1, index=perm) * signs.to(torch.float32)
    n = block
    y = y.reshape(-1, n)
    h = 1
    while h < n:
        y = y.reshape(-1, n // (2 * h), 2, h)
        left, right = y[:, :, 0, :], y[:, :, 1, :]
        y = torch.cat((left + right, left - right), dim=-1).reshape(-1, n)
        h *= 2
    rot = (y * (1.0 / math.sqrt(block))).reshape(x.shape)
    return torch.bucketize(rot, boundaries), norms.reshape(-1)


@pytest.mark.parametrize(("name", "k", "block", "abits", "dtype", "rows", "kind"), CONFIGS)
def test_oracle_codes_differ_from_the_torch_norm_specification_only_at_boundary_ties(name, k, block, abits, dtype, rows, kind):
    gen = torch.Generator().manual_seed(k * 7 + abits)
    perm, signs, h, inv = o.rpbh_constants(k, 0, block)
    _, bounds = reference_tables(k, abits)
    x = make_input(kind, rows, k, dtype, gen)
    want, s_spec = spec_codes(x, torch.from_numpy(perm.astype(np.int64)), torch.from_numpy(signs), torch.from_numpy(bounds), h, 1e-10)
    want = want.numpy().astype(np.uint8)
    got, s_oracle = oracle_c.rotate_quantize(x.float().numpy(), perm, signs, bounds, h, 1e-10, inv)
    differ = np.argwhere(want != got)
    total = want.size
    # a flip needs a coordinate within ~1e-7 relative of one of the boundaries: far below 1e-5 of all codes
    assert len(differ) <= max(3, total * 1e-5), f"{name}: {len(differ)} of {total} codes differ"
    if len(differ) == 0:
        return
    # fp64 recomputation of the rows that hold a difference
    x64 = x.double().numpy()
    s_spec = s_spec.numpy()
    for row in np.unique(differ[:, 0]):
        assert s_spec[row] != s_oracle[row], f"{name}: row {row} has equal norms but different codes"
        exact = float(np.linalg.norm(x64[row]))
        ulp = float(np.spacing(np.float32(exact)))
        # both are fp32 sums of thousands of squares in different orders; the oracle's tree stays within a few
        # ulps of the exact norm, torch's CPU reduction drifts further on long rows (ten ulps at 12288 values)
        assert abs(float(s_oracle[row]) - exact) <= 4 * ulp, f"{name}: the oracle's norm of row {row} is off"
        assert abs(float(s_spec[row]) - exact) <= 64 * ulp, f"{name}: torch's norm of row {row} is off"
        moved = abs(float(s_spec[row]) - float(s_oracle[row])) / exact   # how far the two norms move every coordinate, relatively
        unit = x64[row] / (np.linalg.norm(x64[row]) + 1e-10)
        y = (unit[perm] * signs).reshape(-1, h)
        step = 1
        while step < h:
            y = y.reshape(-1, h // (2 * step), 2, step)
            y = np.concatenate((y[:, :, 0, :] + y[:, :, 1, :], y[:, :, 0, :] - y[:, :, 1, :]), axis=-1).reshape(-1, h)
            step *= 2
        rot = (y / math.sqrt(h)).reshape(-1)
        for col in differ[differ[:, 0] == row][:, 1]:
            a, b = int(want[row, col]), int(got[row, col])
            assert abs(a - b) == 1, f"{name}: codes {a} and {b} at ({row}, {col}) are not neighbours"
            boundary = float(bounds[min(a, b)])
            gap = abs(rot[col] - boundary)
            # a tie: the value sits closer to the boundary than the norms moved it plus fp32 rounding of the rotation
            assert gap <= (moved + 2.0 ** -20) * max(abs(boundary), abs(rot[col]), 1e-30), \
                f"{name}: value {rot[col]!r} at ({row}, {col}) is {gap:.3e} away from boundary {boundary!r}: not a tie"
