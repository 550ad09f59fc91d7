"""The configurations of the benchmark at their full sizes, through the layer's one-call entry
point (which takes the plan-based quantizer for these sizes): EVERY activation code and token
norm must be the oracle's bit for bit (the C oracle quantizes all rows, a few seconds per case
on the host cores), and the outputs of a sample of token rows the oracle's within the path's
bound.  The codebook tables are the reference generator's own (tests/golden/codebooks_v2.json).
The weights are random index bytes (what the matmul reads does not depend on how the indices
were made)."""

from __future__ import annotations

import math

import numpy as np
import pytest
import torch

from oracle import oracle_c, oracle_np as o
from parity_util import cosine, output_error, outside_rounded_bound, reference_tables

pytestmark = pytest.mark.gpu

F32 = np.float32


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


FULL_SIZE = [
    # name, M, K, N, wbits, abits, activation kind
    ("c2 fc1", 2048, 1152, 4608, 4, 4, "outlier_columns"),
    ("c2 fc2", 2048, 4608, 1152, 4, 4, "outlier_columns"),
    ("c3 qkv", 4608, 3072, 9216, 3, 3, "student"),
    ("c3 mlp down", 4608, 12288, 3072, 3, 3, "student"),
    ("c4 fc1", 32760, 5120, 13824, 4, 6, "outliers"),
    ("c4 fc2", 32760, 13824, 5120, 4, 6, "outliers"),
    ("c5 up, 16 tokens", 16, 4096, 14336, 3, 4, "normal"),
    ("c5 down, 1 token", 1, 14336, 4096, 3, 4, "normal"),
    ("c5 q, 1 token", 1, 4096, 4096, 2, 4, "normal"),
]


def activations(kind, m, k, gen):
    x = torch.randn(m, k, generator=gen)
    if kind == "outlier_columns":
        cols = torch.randperm(k, generator=gen)[: max(1, k // 200)]
        x[:, cols] *= 30
    elif kind == "outliers":
        x[torch.rand(m, k, generator=gen) < 0.01] *= 20
    elif kind == "student":
        x = torch.from_numpy(np.random.default_rng(int(gen.initial_seed())).standard_t(4, size=(m, k)).astype(F32))
    return x.to(torch.bfloat16)


@pytest.mark.parametrize(("name", "m", "k", "n", "wbits", "abits", "kind"), FULL_SIZE)
def test_full_size_layer(dev, name, m, k, n, wbits, abits, kind):
    from orbitquant_amd import ops

    gen = torch.Generator().manual_seed(1000 + m + k + n)
    perm, signs, block, inv = o.rpbh_constants(k, 0, "paper")
    ca, ba = reference_tables(k, abits)
    cw, _ = reference_tables(k, wbits)
    packed = torch.randint(0, 256, ((n * k * wbits + 7) // 8,), generator=gen, dtype=torch.uint8)
    r = (0.02 * math.sqrt(k) * (1 + 0.05 * torch.randn(n, generator=gen))).to(torch.bfloat16)
    bias = (0.1 * torch.randn(n, generator=gen)).to(torch.bfloat16)
    x = activations(kind, m, k, gen)

    xd = x.to(dev)
    perm_d, signs_d = torch.from_numpy(perm.astype(np.int32)).to(dev), torch.from_numpy(signs).to(dev)
    ba_d, ca_d, cw_d = torch.from_numpy(ba).to(dev), torch.from_numpy(ca).to(dev), torch.from_numpy(cw).to(dev)
    kw = dict(block_size=block, eps=1e-10, inv_sqrt_block=float(inv))
    plan = ops.rotate_plan(perm_d, signs_d, ba_d, block_size=block, inv_sqrt_block=float(inv))
    out = ops.quantized_linear(xd, perm_d, signs_d, ba_d, ca_d, packed.to(dev), r.to(dev), cw_d, activation_bits=abits,
                               weight_bits=wbits, out_features=n, bias=bias.to(dev), plan=plan, **kw)
    codes, _, norms = ops.rotate_quantize(xd, perm_d, signs_d, ba_d, code_format="u8", plan=plan, **kw)

    # every code and norm of the launch
    want_codes, want_s = oracle_c.rotate_quantize(x.float().numpy(), perm, signs, ba, block, 1e-10, inv)
    got_codes = codes.cpu().numpy()
    mismatches = int(np.count_nonzero(got_codes != want_codes))
    assert mismatches == 0, f"{name}: {mismatches} of {got_codes.size} activation codes differ from the oracle"
    assert np.array_equal(norms.cpu().numpy().view(np.int32), want_s.view(np.int32)), f"{name}: token norms differ from the oracle"
    if m > 16:  # the plain kernel (what launches without a plan run) gives the same codes
        codes_plain, _, norms_plain = ops.rotate_quantize(xd, perm_d, signs_d, ba_d, code_format="u8", **kw)
        assert torch.equal(codes_plain, codes) and torch.equal(norms_plain, norms)
    del got_codes

    rows = np.unique(np.concatenate([[0, m - 1], np.random.default_rng(m).integers(0, m, size=30)]))
    want = oracle_c.linear_from_codes(want_codes[rows], want_s[rows], ca, packed.numpy(), wbits, r.float().numpy(), cw,
                                      bias.float().numpy(), n)
    got = out[rows].float().cpu().numpy()
    strict, rounded = output_error(got, want, want_s[rows], r.float().numpy(), k, True, True)
    assert rounded <= 1.0, f"{name}: max error is {rounded:.3f} of the bound ({strict:.3f} without bf16's half-ulp)"
    # every stored output is the rounding of a value within the stated bound: any excess is the bf16 rounding alone
    bad = outside_rounded_bound(got, want, want_s[rows], r.float().numpy(), k, True)
    assert bad == 0, f"{name}: {bad} outputs are not the rounding of any value within the bound"
    cos = cosine(got, want)
    assert cos >= 0.9999, f"{name}: cosine {cos}"
