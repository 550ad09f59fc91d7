"""GPU tests of the fused output activation: oq_packed_linear_mapped / the output_map of
oq_quantized_linear / OrbitLinear.fuse_output_activation.  The contract is bit identity with
applying the function to the stored result of the plain call."""

from __future__ import annotations

import pytest
import torch

pytestmark = pytest.mark.gpu

gelu = torch.nn.functional.gelu


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


def make_case(dev, m, k, n, wbits, abits, dtype, seed, scale=1.0):
    from orbitquant_amd.codebooks import get_codebook
    from orbitquant_amd.rotations import get_rpbh_rotation

    rot, acb, wcb = get_rpbh_rotation(k, 0, "paper"), get_codebook(k, abits), get_codebook(k, wbits)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    x[torch.rand(m, k, generator=g) < 0.01] *= 20
    return dict(
        x=x.to(dtype).to(dev), perm=rot.permutation.to(torch.int32).to(dev), signs=rot.signs.to(torch.int8).to(dev),
        bounds=acb.boundaries.to(dev), cents=acb.centroids.to(dev), wcents=wcb.centroids.to(dev),
        packed=torch.randint(0, 256, ((n * k * wbits + 7) // 8,), generator=g, dtype=torch.uint8).to(dev),
        # row norms spread over many binades, so that outputs fall inside and outside the LDS window
        rn=(scale * 0.02 * torch.exp(3.0 * torch.randn(n, generator=g))).to(torch.bfloat16).to(dev),
        bias=(0.1 * torch.randn(n, generator=g)).to(dtype).to(dev),
        kw=dict(block_size=rot.block_size, eps=1e-10, inv_sqrt_block=rot.normalization), n=n, k=k, wbits=wbits, abits=abits)


def linear(c, output_map=None):
    from orbitquant_amd import ops

    return ops.quantized_linear(c["x"], c["perm"], c["signs"], c["bounds"], c["cents"], c["packed"], c["rn"],
                                c["wcents"], activation_bits=c["abits"], weight_bits=c["wbits"],
                                out_features=c["n"], bias=c["bias"], output_map=output_map, **c["kw"])


CASES = [
    # m, k, n, wbits, abits, dtype, tile override
    (2048, 1152, 4608, 4, 4, torch.bfloat16, None),    # C2 fc1: 256x192 tiles
    (300, 1152, 1152, 4, 4, torch.bfloat16, "0"),      # ragged M: guarded stores
    (300, 1152, 1152, 4, 4, torch.bfloat16, "1"),
    (515, 1024, 776, 3, 3, torch.bfloat16, "2"),
    (515, 1024, 776, 3, 3, torch.bfloat16, "3"),
    (515, 2304, 1152, 4, 4, torch.bfloat16, "4"),      # K-split kernel: the epilogue runs per wavefront
    (300, 1024, 512, 4, 6, torch.bfloat16, None),      # byte codes
    (300, 1024, 512, 4, 4, torch.float16, None),       # fp16: every value through the full table
    (16, 1024, 512, 4, 4, torch.bfloat16, None),       # streaming kernel + elementwise launch
    (1, 4096, 4096, 3, 4, torch.bfloat16, None),       # one-token launch + elementwise launch
    (40, 1100, 96, 4, 4, torch.bfloat16, None),        # shape-agnostic kernel + elementwise launch
    (64, 512, 100, 4, 4, torch.bfloat16, None),        # N % 8 != 0: shape-agnostic kernel
]


@pytest.mark.parametrize(("m", "k", "n", "wbits", "abits", "dtype", "tile"), CASES)
@pytest.mark.parametrize("fn", [gelu, torch.nn.functional.silu])
def test_output_map_equals_function_of_plain_output(dev, m, k, n, wbits, abits, dtype, tile, fn, library_switch):
    from orbitquant_amd import ops

    if tile is not None:
        library_switch("OQ_GEMM_TILE", tile)
    c = make_case(dev, m, k, n, wbits, abits, dtype, seed=m + k + n)
    table = ops.activation_table(fn, dtype, dev)
    plain = linear(c)
    assert torch.isfinite(plain.float()).all()
    assert torch.equal(linear(c, output_map=table), fn(plain))


@pytest.mark.parametrize("m,k,n,splits", [(200, 2048, 256, "2"), (128, 8192, 520, "8"), (48, 2048, 256, None)])
def test_output_map_behind_shared_k_and_row_blocks(dev, m, k, n, splits, library_switch):
    """The map after a GEMM that shares K between workgroups (applied by a launch of its own, after the parts
    are added) and after the streaming kernel at 17 to 64 tokens."""
    from orbitquant_amd import ops

    if splits is not None:
        library_switch("OQ_GEMM_WG_SPLIT", splits)
    c = make_case(dev, m, k, n, 4, 4, torch.bfloat16, seed=m + k + n)
    table = ops.activation_table(gelu, torch.bfloat16, dev)
    plain = linear(c)
    assert torch.isfinite(plain.float()).all()
    assert torch.equal(linear(c, output_map=table), gelu(plain))


def test_packed_linear_mapped_entry_point(dev):
    from orbitquant_amd import _lib, ops

    c = make_case(dev, 200, 512, 256, 4, 4, torch.bfloat16, seed=9)
    table = ops.activation_table(gelu, torch.bfloat16, dev)
    codes, _, norms = ops.rotate_quantize(c["x"], c["perm"], c["signs"], c["bounds"], code_format="nibble", **c["kw"])
    kw = dict(code_format="nibble", activation_bits=4, weight_bits=4, out_features=256, in_features=512, bias=c["bias"])
    plain = ops.packed_linear(codes, norms, c["cents"], c["packed"], c["rn"], c["wcents"], **kw)
    assert torch.equal(ops.packed_linear(codes, norms, c["cents"], c["packed"], c["rn"], c["wcents"], output_map=table, **kw),
                       gelu(plain))
    with pytest.raises(ValueError):   # fp32 outputs have no table
        ops.packed_linear(codes, norms, c["cents"], c["packed"], c["rn"], c["wcents"], output_map=table,
                          output_dtype=torch.float32, **{**kw, "bias": None})
    lib = _lib.load()
    out = torch.empty(200, 256, dtype=torch.float32, device=dev)
    args = (codes.data_ptr(), 1, norms.data_ptr(), c["cents"].data_ptr(), 4, c["packed"].data_ptr(), 4, c["rn"].data_ptr(),
            c["wcents"].data_ptr(), None, 0, 200, 256, 512, out.data_ptr())
    assert lib.oq_packed_linear_mapped(*args, 0, table.data_ptr(), None, 0, None) == 1      # fp32 output
    assert lib.oq_packed_linear_mapped(*args, 2, None, None, 0, None) == 1                  # null table
    torch.cuda.synchronize()


@pytest.mark.parametrize("m", [1, 16, 2048])
def test_fused_output_activation_layer(dev, m):
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(21)
    cfg = recipe("w4a4")
    fc1 = OrbitLinear.from_linear(torch.nn.Linear(256, 1024), config=cfg).to(dev).to(torch.bfloat16)
    fc2 = OrbitLinear.from_linear(torch.nn.Linear(1024, 256), config=cfg).to(dev).to(torch.bfloat16)
    x = torch.randn(m, 256, dtype=torch.bfloat16, device=dev)
    want = fc2(gelu(fc1(x)))
    fc1.fuse_output_activation(gelu, dtype=torch.bfloat16)
    mlp = torch.nn.Sequential(fc1, fc2)
    assert torch.equal(mlp(x), want)
    assert torch.equal(torch.compile(mlp, fullgraph=True)(x), want)
    with pytest.raises(ValueError):
        fc1(x.float())
    fc1.fuse_output_activation(None)
    assert torch.equal(fc2(gelu(fc1(x))), want)
