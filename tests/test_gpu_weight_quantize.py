"""GPU tests of oq_quantize_weight (the weight side of a layer made on the device): the packed
index stream and the bf16 row norms must equal the oracle's (`oracle_np.quantize_weight` with the
kernel's summation order for the row norm) byte for byte, for the five recipes at the reference's
own test dimension, at the configuration dimensions, for every packing width and input dtype,
with zero rows, and whatever the row tiling.  Against the oracle with torch's norm (the
reference's host path) the norms must agree after bf16 rounding almost everywhere and the
indices everywhere except at boundary ties."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import oracle_np as o
from parity_util import reference_tables

pytestmark = pytest.mark.gpu

RECIPES = {"w4a4": (4, 4), "w3a3": (3, 3), "w2a4": (2, 4), "w2a3": (2, 3), "w4a6": (4, 6)}


@pytest.fixture(scope="module")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("needs an AMD GPU")
    from orbitquant_amd import _lib

    lib = _lib.load()
    assert lib.oq_device_ok() == 0, lib.oq_last_error()
    return torch.device("cuda:0")


def gpu_quantize(dev, w, perm, signs, bounds, block, inv, bits, row_tile=None):
    from orbitquant_amd import ops

    return ops.quantize_weight(w.to(dev), torch.from_numpy(perm.astype(np.int32)).to(dev), torch.from_numpy(signs).to(dev),
                               torch.from_numpy(bounds).to(dev), bits=bits, block_size=block, eps=1e-10,
                               inv_sqrt_block=float(inv), row_tile=row_tile)


@pytest.mark.parametrize("recipe", sorted(RECIPES))
def test_five_recipes_at_the_reference_test_dimension(dev, recipe):
    # tests/test_paper_reference_oracle.py:122-203 of the reference: dim 24 (block 8), seed 29
    wbits, _ = RECIPES[recipe]
    k, n = 24, 13
    perm, signs, block, inv = o.rpbh_constants(k, 29, "paper")
    _, bounds = reference_tables(k, wbits)
    w = torch.randn(n, k, generator=torch.Generator().manual_seed(29))
    w[4] = 0
    packed, norms = gpu_quantize(dev, w, perm, signs, bounds, block, inv, wbits)
    want_packed, want_norms, _ = o.quantize_weight(w.numpy(), perm, signs, bounds, block, 1e-10, wbits, norm_order="sumsq_v1")
    assert np.array_equal(packed.cpu().numpy(), want_packed)
    assert torch.equal(norms.cpu(), want_norms)
    assert float(norms[4]) == 0.0
    # the host path of the product (torch's norm) on this small case: identical
    host_packed, host_norms, _ = o.quantize_weight(w.numpy(), perm, signs, bounds, block, 1e-10, wbits)
    assert np.array_equal(packed.cpu().numpy(), host_packed) and torch.equal(norms.cpu(), host_norms)


@pytest.mark.parametrize(("n", "k", "bits", "dtype"), [
    (4608, 1152, 4, torch.float32),    # c2 fc1
    (1152, 4608, 4, torch.bfloat16),   # c2 fc2
    (1024, 3072, 3, torch.float32),    # c3 (a slab of rows)
    (512, 12288, 3, torch.float16),    # c3 fc2, block 4096
    (512, 5120, 4, torch.bfloat16),    # c4 fc1
    (256, 13824, 4, torch.float32),    # c4 fc2
    (1024, 4096, 2, torch.float32),    # c5 q / k
    (512, 14336, 3, torch.bfloat16),   # c5 down, block 2048
    (300, 1152, 6, torch.float32),
    (77, 2048, 8, torch.float32),
    (64, 1024, 1, torch.float32),
    (50, 520, 5, torch.float32),       # ragged row length, block 8
])
def test_configuration_dimensions(dev, n, k, bits, dtype):
    perm, signs, block, inv = o.rpbh_constants(k, 0, "paper")
    _, bounds = reference_tables(k, bits) if bits in (2, 3, 4, 6, 8) else o.lloyd_max_tables(k, bits)
    gen = torch.Generator().manual_seed(n + k + bits)
    w = (torch.randn(n, k, generator=gen) * 0.02).to(dtype)
    w[n // 3] = 0
    w[n // 2, ::3] *= 40
    packed, norms = gpu_quantize(dev, w, perm, signs, bounds, block, inv, bits)
    want_packed, want_norms, want_idx = o.quantize_weight(w.float().numpy(), perm, signs, bounds, block, 1e-10, bits,
                                                         norm_order="sumsq_v1")
    assert torch.equal(norms.cpu(), want_norms)
    got_idx = o.unpack_bits(packed.cpu().numpy(), bits, n * k).reshape(n, k)
    assert int(np.count_nonzero(got_idx != want_idx)) == 0
    assert np.array_equal(packed.cpu().numpy(), want_packed)
    # row tiling writes the same stream
    tiled, tiled_norms = gpu_quantize(dev, w, perm, signs, bounds, block, inv, bits, row_tile=37 if (37 * k * bits) % 8 == 0 else 40)
    assert torch.equal(tiled, packed) and torch.equal(tiled_norms, norms)
    # against torch's norm: the same up to ties
    host_packed, host_norms, host_idx = o.quantize_weight(w.float().numpy(), perm, signs, bounds, block, 1e-10, bits)
    assert int((norms.cpu().view(torch.int16) != host_norms.view(torch.int16)).sum()) <= max(1, n // 500)
    assert int(np.count_nonzero(got_idx != host_idx)) <= max(2, n * k // 200000)


def test_layer_built_from_a_gpu_weight_matches_the_host_built_layer(dev):
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(3)
    lin = torch.nn.Linear(1152, 384)
    host = OrbitLinear.from_linear(lin, config=recipe("w4a4"))
    device_built = OrbitLinear.from_linear(lin.to(dev), config=recipe("w4a4"))
    assert device_built.packed_weight_indices.device.type == "cuda"
    assert torch.equal(device_built.row_norms.cpu(), host.row_norms)
    differing = int((device_built.packed_weight_indices.cpu() != host.packed_weight_indices).sum())
    assert differing <= 2   # ties only (the two paths sum a row's squares in different orders)
    x = torch.randn(64, 1152, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).to(dev)
    y_dev = device_built(x)
    y_host = host.to(dev)(x)
    assert float((y_dev.float() - y_host.float()).abs().max()) <= 0.05 * float(y_host.float().abs().max())


def test_argument_checks(dev):
    from orbitquant_amd import _lib

    lib = _lib.load()
    w = torch.zeros(4, 1024, device=dev)
    bounds = torch.zeros(15, device=dev)
    plan = torch.zeros(int(lib.oq_rotate_plan_bytes(1024)), dtype=torch.uint8, device=dev)
    packed = torch.zeros(4 * 1024 // 2, dtype=torch.uint8, device=dev)
    norms = torch.zeros(4, dtype=torch.bfloat16, device=dev)

    def call(k=1024, block=256, bits=4, levels=16, w_ptr=None):
        return lib.oq_quantize_weight(w.data_ptr() if w_ptr is None else w_ptr, 0, 4, k, plan.data_ptr(), bounds.data_ptr(), levels,
                                      block, 1e-10, 0.0625, bits, packed.data_ptr(), norms.data_ptr(), None)

    assert call(bits=9) == 1 and call(levels=17) == 1 and call(block=48) == 1
    assert call(k=1020, block=4) == 2      # block below 8: no kernel
    assert call(block=4) == 2
    assert call(w_ptr=w.data_ptr() + 4) == 1
    assert call() == 0                      # a zero plan has the wrong magic: no indices are written, the row norms are NaN
    torch.cuda.synchronize()
    assert not packed.any() and bool(torch.isnan(norms.float()).all())
