"""GPU tests of the fused input activation: oq_rotate_quantize_mapped and OrbitLinear.fuse_input_activation.

The contract is bit identity: quantizing x through the table of an elementwise function f
returns exactly what quantizing the tensor f(x) returns (codes, norms, values), and so a
layer with a fused input activation returns exactly what the layer returns on f(x).  The
unmapped kernel is pinned to the oracle elsewhere; one case here is checked against the
oracle directly as well.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import oracle_c, oracle_np as o

pytestmark = pytest.mark.gpu

gelu = torch.nn.functional.gelu


def gelu_tanh(t):
    return torch.nn.functional.gelu(t, approximate="tanh")


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


def rotation_and_tables(k, abits, dev, block="paper"):
    perm, signs, blk, inv = o.rpbh_constants(k, 0, block)
    cents, bounds = o.lloyd_max_tables(k, abits)
    return dict(
        perm_np=perm, signs_np=signs, bounds_np=bounds, block=blk, inv=inv,
        perm=torch.from_numpy(perm.astype(np.int32)).to(dev), signs=torch.from_numpy(signs).to(dev),
        bounds=torch.from_numpy(bounds).to(dev), cents=torch.from_numpy(cents).to(dev))


def make_input(m, k, dtype, scale, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g) * scale
    x[torch.rand(m, k, generator=g) < 0.01] *= 20
    # values outside the 16 binades the kernel keeps in LDS, zeros of both signs, and the largest finite inputs
    special = torch.tensor([0.0, -0.0, 1e-20, -1e-20, 300.0, -300.0, 1e-4, -1e-4, 6e4, -6e4, 2.0 ** -10, -(2.0 ** 6)])
    x[0, : special.numel()] = special
    x[m - 1, k - special.numel():] = special
    return x.to(dtype)


MAP_CASES = [
    # m, k, abits, dtype, code_format, values, fn, scale
    (64, 4608, 4, torch.bfloat16, "nibble", None, gelu, 1.6),          # 16-bit staging, three passes
    (300, 1152, 4, torch.bfloat16, "nibble", None, gelu, 1.0),         # three wavefronts per row
    (33, 12288, 3, torch.bfloat16, "nibble", None, gelu, 1.0),         # block 4096: stages through LDS
    (5, 14336, 4, torch.bfloat16, "u8", "unit_bf16", gelu, 1.0),       # several pass groups (few rows)
    (37, 1100, 4, torch.bfloat16, "u8", "scaled", gelu, 1.0),          # K % 8 != 0: element-wise loads
    (64, 4608, 4, torch.float16, "nibble", None, gelu, 1.6),           # fp16: every input through the full table
    (40, 5120, 6, torch.float16, "u8", None, torch.nn.functional.silu, 1.0),
    (64, 4608, 4, torch.bfloat16, "nibble", None, gelu, 1e-3),         # mostly below the LDS window
    (64, 2048, 4, torch.bfloat16, "nibble", None, gelu_tanh, 40.0),    # mostly above / saturated
    (17, 3072, 3, torch.bfloat16, "nibble", None, torch.relu, 1.0),    # half the outputs are zero
]


@pytest.mark.parametrize(("m", "k", "abits", "dtype", "fmt", "values", "fn", "scale"), MAP_CASES)
def test_mapped_quantizer_equals_quantizer_of_mapped_tensor(dev, m, k, abits, dtype, fmt, values, fn, scale):
    from orbitquant_amd import ops

    c = rotation_and_tables(k, abits, dev)
    x = make_input(m, k, dtype, scale, seed=m + k).to(dev)
    table = ops.activation_table(fn, dtype, dev)
    kw = dict(block_size=c["block"], eps=1e-10, inv_sqrt_block=float(c["inv"]), centroids=c["cents"],
              code_format=fmt, values=values)
    want = ops.rotate_quantize(fn(x), c["perm"], c["signs"], c["bounds"], **kw)
    got = ops.rotate_quantize(x, c["perm"], c["signs"], c["bounds"], input_map=table, **kw)
    for name, a, b in zip(("codes", "values", "norms"), got, want):
        if b is None:
            assert a is None
        else:
            assert torch.equal(a, b), f"{name} differ"


PLAN_MAP_CASES = [
    # m, k, abits, code_format, fn, scale, block: bf16 rows into codes, the forms the plan-based kernel takes with a map
    (2048, 4608, 4, "nibble", gelu, 1.6, "paper"),     # the MLP pair's second quantizer (three passes, nine units)
    (300, 1152, 4, "nibble", gelu, 1.0, "paper"),      # lanes past the row's end in the last pass
    (64, 4608, 4, "u8", gelu, 1e-3, "paper"),          # most values below the window: the table in memory
    (33, 12288, 3, "nibble", gelu_tanh, 40.0, "paper"),  # block 4096, saturated values
    (100, 3072, 6, "u8", torch.nn.functional.silu, 1.0, 64),
    (17, 2048, 4, "nibble", torch.relu, 1.0, 8),       # the smallest block; half the mapped values are zero
]


@pytest.mark.parametrize(("m", "k", "abits", "fmt", "fn", "scale", "block"), PLAN_MAP_CASES)
def test_mapped_plan_kernel_equals_plan_kernel_on_the_mapped_tensor(dev, m, k, abits, fmt, fn, scale, block):
    """With a rotate plan the mapped quantizer runs the plan-based kernel (the table's window in LDS, every
    value looked up as the row is read); its codes and norms are those of the same kernel on f(x), and of
    the plain kernel through the map, bit for bit."""
    from orbitquant_amd import ops

    c = rotation_and_tables(k, abits, dev, block)
    x = make_input(m, k, torch.bfloat16, scale, seed=3 * m + k).to(dev)
    table = ops.activation_table(fn, torch.bfloat16, dev)
    levels = c["bounds"].numel() + 1
    plan = ops.rotate_plan(c["perm"], c["signs"], c["bounds"], block_size=c["block"], inv_sqrt_block=float(c["inv"]))
    kw = dict(block_size=c["block"], eps=1e-10, inv_sqrt_block=float(c["inv"]), code_format=fmt)
    want = ops.rotate_quantize(fn(x), c["perm"], c["signs"], c["bounds"], plan=plan, **kw)
    plain = ops.rotate_quantize(x, c["perm"], c["signs"], c["bounds"], input_map=table, **kw)
    got = ops.rotate_quantize(x, c["perm"], c["signs"], c["bounds"], input_map=table, plan=plan, **kw)
    assert levels == 1 << abits
    for name, a, b, p in zip(("codes", "values", "norms"), got, want, plain):
        if b is not None:
            assert torch.equal(a, b), f"{name} differ from the plan kernel on f(x)"
            assert torch.equal(a, p), f"{name} differ from the plain kernel through the map"


def test_mapped_quantizer_against_the_oracle(dev):
    from orbitquant_amd import ops

    m, k, abits = 48, 4608, 4
    c = rotation_and_tables(k, abits, dev)
    x = make_input(m, k, torch.bfloat16, 1.6, seed=7).to(dev)
    table = ops.activation_table(gelu, torch.bfloat16, dev)
    codes, _, norms = ops.rotate_quantize(x, c["perm"], c["signs"], c["bounds"], block_size=c["block"], eps=1e-10,
                                          inv_sqrt_block=float(c["inv"]), code_format="u8", input_map=table)
    fx = gelu(x).float().cpu().numpy()
    want_codes, want_s = oracle_c.rotate_quantize(fx, c["perm_np"], c["signs_np"], c["bounds_np"], c["block"], 1e-10, c["inv"])
    assert np.array_equal(codes.cpu().numpy(), want_codes)
    assert np.array_equal(norms.cpu().numpy(), want_s)


def test_activation_table_is_the_function_on_every_bit_pattern(dev):
    from orbitquant_amd import ops

    for dtype in (torch.bfloat16, torch.float16):
        table = ops.activation_table(gelu, dtype, dev)
        bits = torch.arange(65536, dtype=torch.int32, device=dev).to(torch.int16)
        want = gelu(bits.view(dtype))
        assert torch.equal(table.view(torch.int16), want.view(torch.int16))


def test_mapped_quantizer_rejects_bad_arguments(dev):
    from orbitquant_amd import _lib, ops

    c = rotation_and_tables(512, 4, dev)
    table = ops.activation_table(gelu, torch.bfloat16, dev)
    kw = dict(block_size=c["block"], eps=1e-10, inv_sqrt_block=float(c["inv"]))
    with pytest.raises(ValueError):   # fp32 inputs have no 65536-entry table
        ops.rotate_quantize(torch.randn(4, 512, device=dev), c["perm"], c["signs"], c["bounds"], input_map=table, **kw)
    with pytest.raises(ValueError):   # table of another dtype
        ops.rotate_quantize(torch.randn(4, 512, device=dev).half(), c["perm"], c["signs"], c["bounds"], input_map=table, **kw)
    with pytest.raises(ValueError):
        ops.activation_table(gelu, torch.float32, dev)
    # the C entry point itself: null table, fp32 dtype
    lib = _lib.load()
    x = torch.randn(4, 512, device=dev)
    codes = torch.empty(4, 512, dtype=torch.uint8, device=dev)
    norms = torch.empty(4, device=dev)
    args = (4, 512, c["perm"].data_ptr(), c["signs"].data_ptr(), c["bounds"].data_ptr(), None, 16, c["block"], 1e-10,
            float(c["inv"]), None, codes.data_ptr(), 0, None, 0, norms.data_ptr(), None)
    assert lib.oq_rotate_quantize_mapped(x.data_ptr(), 2, None, *args) == 1
    assert lib.oq_rotate_quantize_mapped(x.data_ptr(), 0, table.data_ptr(), *args) == 1
    assert b"16-bit" in lib.oq_last_error()
    torch.cuda.synchronize()


@pytest.mark.parametrize(("recipe_name", "m"), [("w4a4", 2048), ("w4a4", 8), ("w3a3", 300), ("w4a6", 64)])
def test_fused_input_activation_layer_is_bit_identical(dev, recipe_name, m):
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(11)
    cfg = recipe(recipe_name)
    fc1 = OrbitLinear.from_linear(torch.nn.Linear(256, 1024), config=cfg).to(dev).to(torch.bfloat16)
    fc2 = OrbitLinear.from_linear(torch.nn.Linear(1024, 256), config=cfg).to(dev).to(torch.bfloat16)
    x = torch.randn(m, 256, dtype=torch.bfloat16, device=dev)
    h = fc1(x)
    want = fc2(gelu(h))
    fc2.fuse_input_activation(gelu, dtype=torch.bfloat16)
    assert torch.equal(fc2(h), want)
    with pytest.raises(ValueError):
        fc2(h.float())
    # the table survives a dtype cast of the module bit for bit
    fc2.to(torch.bfloat16)
    assert torch.equal(fc2(h), want)
    fc2.fuse_input_activation(None)
    assert torch.equal(fc2(gelu(h)), want)


def test_fused_input_activation_under_torch_compile(dev):
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(12)
    cfg = recipe("w4a4")
    fc1 = OrbitLinear.from_linear(torch.nn.Linear(512, 1024), config=cfg).to(dev)
    fc2 = OrbitLinear.from_linear(torch.nn.Linear(1024, 512), config=cfg).to(dev)
    x = torch.randn(3, 20, 512, dtype=torch.bfloat16, device=dev)
    want = fc2(gelu(fc1(x)))
    fc2.fuse_input_activation(gelu, dtype=torch.bfloat16)
    mlp = torch.nn.Sequential(fc1, fc2)
    assert torch.equal(mlp(x), want)
    assert torch.equal(torch.compile(mlp, fullgraph=True)(x), want)
