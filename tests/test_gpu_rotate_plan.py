"""GPU tests of the plan-based rotate+quantize kernel (oq_rotate_plan_build + the rotate_plan
argument of oq_rotate_quantize): codes, norms and values must equal the CPU oracle bit for bit,
and therefore the plain kernel, on every configuration dimension, every block size the kernel is
instantiated for, every output form, and on rows that take its slow paths (tiny or non-finite
values, codebooks without a cell table)."""

from __future__ import annotations

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


def constants(dev, k, block, bits):
    from oracle import oracle_np

    perm, signs, h, inv = oracle_np.rpbh_constants(k, 0, block)
    from parity_util import reference_tables

    cents, bounds = reference_tables(k, bits)
    t = dict(perm=torch.from_numpy(perm.astype(np.int32)).to(dev), signs=torch.from_numpy(signs.astype(np.int8)).to(dev),
             bounds=torch.from_numpy(bounds).to(dev), cents=torch.from_numpy(cents).to(dev))
    return perm, signs, h, inv, cents, bounds, t


def both_kernels(x, t, h, inv, **kw):
    from orbitquant_amd import ops

    plan = ops.rotate_plan(t["perm"], t["signs"], t["bounds"], block_size=h, inv_sqrt_block=float(inv))
    fast = ops.rotate_quantize(x, t["perm"], t["signs"], t["bounds"], block_size=h, eps=1e-10, inv_sqrt_block=float(inv),
                               plan=plan, **kw)
    plain = ops.rotate_quantize(x, t["perm"], t["signs"], t["bounds"], block_size=h, eps=1e-10, inv_sqrt_block=float(inv), **kw)
    return fast, plain


def make_rows(m, k, dtype, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    x[torch.rand(m, k, generator=g) < 0.01] *= 20
    x[3] = 0
    x[5, ::2] = 0
    return x.to(dtype)


CONFIG_DIMS = [(1152, 64), (1152, "paper"), (4608, "paper"), (3072, "paper"), (12288, "paper"), (5120, "paper"),
               (13824, "paper"), (4096, "paper"), (14336, "paper")]


@pytest.mark.parametrize("k,block", CONFIG_DIMS)
@pytest.mark.parametrize("dtype,bits", [(torch.bfloat16, 4), (torch.float16, 3), (torch.float32, 4), (torch.bfloat16, 6)])
def test_plan_kernel_equals_oracle_on_config_dims(dev, k, block, dtype, bits):
    from oracle import oracle_c

    perm, signs, h, inv, cents, bounds, t = constants(dev, k, block, bits)
    m = 37
    x = make_rows(m, k, dtype, seed=k + bits)
    (codes, _, norms), (codes_plain, _, norms_plain) = both_kernels(x.to(dev), t, h, inv, code_format="u8")
    want_codes, want_norms = oracle_c.rotate_quantize(x.float().numpy(), perm, signs, bounds, h, 1e-10, inv)
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(norms.cpu().numpy().view(np.int32), want_norms.view(np.int32))
    assert torch.equal(codes, codes_plain) and torch.equal(norms, norms_plain)


@pytest.mark.parametrize("log_h", range(3, 13))
def test_every_block_size(dev, log_h):
    from oracle import oracle_c

    h = 1 << log_h
    k = max(h, 8) * 3
    for dtype in (torch.bfloat16, torch.float32):
        perm, signs, hh, inv, cents, bounds, t = constants(dev, k, h, 4)
        x = make_rows(19, k, dtype, seed=log_h)
        (packed, _, norms), (packed_plain, _, _) = both_kernels(x.to(dev), t, h, inv, code_format="nibble")
        want_codes, want_norms = oracle_c.rotate_quantize(x.float().numpy(), perm, signs, bounds, h, 1e-10, inv)
        want_packed = (want_codes[:, 0::2] | (want_codes[:, 1::2] << 4)).astype(np.uint8)
        assert np.array_equal(packed.cpu().numpy(), want_packed), (h, dtype)
        assert np.array_equal(norms.cpu().numpy().view(np.int32), want_norms.view(np.int32))
        assert torch.equal(packed, packed_plain)


@pytest.mark.parametrize("k,h", [(520, 8), (1048, 8), (2056, 8), (24 * 64, 64), (17 * 128, 128), (9 * 256, 256)])
def test_ragged_rows(dev, k, h):
    """Rows that are not a multiple of 512: the last unit has idle lanes."""
    from oracle import oracle_c

    perm, signs, hh, inv, cents, bounds, t = constants(dev, k, h, 4)
    x = make_rows(33, k, torch.bfloat16, seed=k)
    (codes, _, norms), _ = both_kernels(x.to(dev), t, h, inv, code_format="u8")
    want_codes, want_norms = oracle_c.rotate_quantize(x.float().numpy(), perm, signs, bounds, h, 1e-10, inv)
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(norms.cpu().numpy().view(np.int32), want_norms.view(np.int32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_rows_that_take_the_ieee_division(dev, dtype):
    """Tiny values, tiny and huge norms, infinities and NaNs: the row-level test must send these
    rows to the plain division, and the result must still be the specification's."""
    from oracle import oracle_c

    k, h = 1024, 256
    perm, signs, hh, inv, cents, bounds, t = constants(dev, k, h, 4)
    x = make_rows(40, k, torch.float32, seed=1)
    tiny = 1e-30 if dtype != torch.float16 else 6e-8
    x[1, 7] = tiny                      # one tiny value in an ordinary row
    x[2] *= 1e-28 if dtype != torch.float16 else 1e-4   # a row of tiny values
    x[4] *= 1e12 if dtype != torch.float16 else 30.0    # a huge norm
    x[6, 100] = float("inf")
    x[7, 5] = float("nan")
    x[8] = 0
    x[8, 9] = -tiny
    if dtype == torch.bfloat16:
        x[9, 3] = 1e-39                 # a bf16 denormal
    x = x.to(dtype)
    (codes, _, norms), (codes_plain, _, norms_plain) = both_kernels(x.to(dev), t, h, inv, code_format="u8")
    with np.errstate(all="ignore"):
        want_codes, want_norms = oracle_c.rotate_quantize(x.float().numpy(), perm, signs, bounds, h, 1e-10, inv)
    assert torch.equal(codes, codes_plain)
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    got = norms.cpu().numpy()
    assert np.array_equal(np.isnan(got), np.isnan(want_norms))
    ok = ~np.isnan(want_norms)
    assert np.array_equal(got[ok].view(np.int32), want_norms[ok].view(np.int32))


@pytest.mark.parametrize("levels", [2, 3, 5, 16, 64, 100, 256])
def test_any_codebook_size_and_awkward_boundaries(dev, levels):
    """Boundary sets for which no cell table exists (more than 64 levels, clustered boundaries)
    take the binary search over the folded thresholds."""
    from oracle import oracle_np

    k, h = 2048, 512
    perm, signs, hh, inv = oracle_np.rpbh_constants(k, 0, h)
    g = np.random.default_rng(levels)
    bounds = np.sort(g.normal(0, 0.03, levels - 1)).astype(np.float32)
    if levels == 16:
        bounds[5] = np.nextafter(bounds[4], np.float32(1))  # two boundaries one ulp apart
    t = dict(perm=torch.from_numpy(perm.astype(np.int32)).to(dev), signs=torch.from_numpy(signs.astype(np.int8)).to(dev),
             bounds=torch.from_numpy(bounds).to(dev))
    x = make_rows(21, k, torch.bfloat16, seed=levels)
    (codes, _, _), (codes_plain, _, _) = both_kernels(x.to(dev), t, h, inv, code_format="u8")
    want, _ = oracle_np.quantize_codes(x.float().numpy(), perm, signs, bounds, h, 1e-10, inv)
    assert np.array_equal(codes.cpu().numpy(), want)
    assert torch.equal(codes, codes_plain)


def test_values_on_exact_boundaries(dev):
    """A rotated value that lands exactly on a boundary belongs to the lower code; the folded
    thresholds must keep that for a factor that is not a power of two (block 512)."""
    from oracle import oracle_np

    k, h = 512, 512
    perm, signs, hh, inv = oracle_np.rpbh_constants(k, 0, h)
    x = np.zeros((64, k), np.float32)
    x[np.arange(64), np.arange(64) * 7 % k] = 1.0   # one-hot rows: every rotated value is +-1/sqrt(512) exactly
    rot = np.float32(1.0) * np.float32(inv)
    bounds = np.array([-rot, np.nextafter(-rot, np.float32(0)), 0.0, np.nextafter(rot, np.float32(0)), rot], np.float32)
    t = dict(perm=torch.from_numpy(perm.astype(np.int32)).to(dev), signs=torch.from_numpy(signs.astype(np.int8)).to(dev),
             bounds=torch.from_numpy(bounds).to(dev))
    (codes, _, _), (codes_plain, _, _) = both_kernels(torch.from_numpy(x).to(dev), t, h, inv, code_format="u8")
    want, _ = oracle_np.quantize_codes(x, perm, signs, bounds, h, 1e-10, inv)
    assert set(np.unique(want)) == {0, 4}   # -rot is not above the boundary -rot: code 0; +rot is above four: code 4
    assert np.array_equal(codes.cpu().numpy(), want) and torch.equal(codes, codes_plain)


@pytest.mark.parametrize("values", ["scaled", "unit_bf16"])
def test_value_outputs(dev, values):
    k, h = 3072, 1024
    perm, signs, hh, inv, cents, bounds, t = constants(dev, k, h, 4)
    for dtype in (torch.bfloat16, torch.float32):
        x = make_rows(23, k, dtype, seed=2).to(dev)
        fast, plain = both_kernels(x, t, h, inv, code_format="u8", values=values, centroids=t["cents"])
        for a, b in zip(fast, plain):
            assert torch.equal(a, b)
        fast, plain = both_kernels(x, t, h, inv, code_format=None, values=values, centroids=t["cents"])
        assert fast[0] is None and torch.equal(fast[1], plain[1]) and torch.equal(fast[2], plain[2])


def test_plan_for_another_shape_is_loud(dev):
    from orbitquant_amd import ops

    perm, signs, h, inv, cents, bounds, t = constants(dev, 1024, 256, 4)
    other = constants(dev, 1024, 512, 4)
    wrong = ops.rotate_plan(other[6]["perm"], other[6]["signs"], other[6]["bounds"], block_size=512, inv_sqrt_block=float(other[3]))
    x = make_rows(32, 1024, torch.bfloat16, seed=3).to(dev)
    lib_codes = torch.full((32, 1024), 0xAB, dtype=torch.uint8, device=dev)
    from orbitquant_amd import _lib

    lib = _lib.load()
    norms = torch.full((32,), -1.0, device=dev)
    rc = lib.oq_rotate_quantize(x.data_ptr(), 2, 32, 1024, t["perm"].data_ptr(), t["signs"].data_ptr(), t["bounds"].data_ptr(),
                                None, 16, 256, 1e-10, float(inv), wrong.data_ptr(), lib_codes.data_ptr(), 0, None, 0,
                                norms.data_ptr(), None)
    torch.cuda.synchronize()
    assert rc == 0
    # the kernel does not walk a plan built for another block size: no codes, and NaN norms, so that
    # whatever is computed from this call's outputs is NaN instead of looking like a result
    assert bool((lib_codes == 0xAB).all()) and bool(torch.isnan(norms).all())
    # the Python wrapper knows what the plan was built for and refuses it before any launch
    with pytest.raises(ValueError, match="rotate plan was built for"):
        ops.rotate_quantize(x, t["perm"], t["signs"], t["bounds"], block_size=256, eps=1e-10, inv_sqrt_block=float(inv),
                            code_format="u8", plan=wrong)


def test_layer_uses_the_plan_and_matches_the_two_call_path(dev):
    from orbitquant_amd import OrbitLinear, ops, recipe

    torch.manual_seed(0)
    lin = torch.nn.Linear(1152, 256)
    layer = OrbitLinear.from_linear(lin, config=recipe("w4a4")).to(dev)
    assert layer._rotation_plan is not None and layer._rotation_plan.device.type == "cuda"
    x = make_rows(300, 1152, torch.bfloat16, seed=4).to(dev)
    y = layer(x)
    codes, _, norms = ops.rotate_quantize(x, layer._rotation_permutation, layer._rotation_signs,
                                          layer._activation_codebook_boundaries, block_size=layer.rotation.block_size,
                                          eps=layer.activation_eps, inv_sqrt_block=layer.rotation.normalization,
                                          code_format="nibble")
    want = ops.packed_linear(codes, norms, layer._activation_codebook_centroids, layer.packed_weight_indices,
                             layer.row_norms, layer._weight_codebook_centroids, code_format="nibble", activation_bits=4,
                             weight_bits=4, out_features=256, in_features=1152, bias=layer.bias.to(torch.bfloat16),
                             output_dtype=torch.bfloat16)
    assert torch.equal(y, want)
