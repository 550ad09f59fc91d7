"""GPU tests of the four-bit copy that 2- and 3-bit layers hand the tile kernel for many-token
calls (`OrbitLinear._matmul_weight`): same indices, same operand values, so the same outputs as the
stored bit stream gives; built lazily, dropped when the weights change or move."""

from __future__ import annotations

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


def make_layer(dev, k, n, wbits, abits, bias=True, seed=0):
    from orbitquant_amd import OrbitLinear, OrbitQuantConfig

    torch.manual_seed(seed)
    return OrbitLinear.from_linear(torch.nn.Linear(k, n, bias=bias), config=OrbitQuantConfig(weight_bits=wbits, activation_bits=abits)).to(dev)


@pytest.mark.parametrize("k,n,wbits,abits,m", [
    (1152, 1152, 3, 3, 512), (1024, 600, 2, 4, 300), (3072, 1024, 3, 3, 4608), (512, 200, 3, 6, 257),
    (1088, 96, 2, 3, 256), (2048, 4096, 3, 4, 1000), (4096, 520, 3, 4, 65), (1024, 256, 2, 4, 100)])
def test_copy_gives_the_outputs_of_the_stored_stream(dev, k, n, wbits, abits, m):
    from orbitquant_amd import ops

    layer = make_layer(dev, k, n, wbits, abits, seed=k + n)
    x = torch.randn(m, k, device=dev, dtype=torch.bfloat16)
    layer.nibble_copy_for_many_tokens = False
    want = layer(x)
    assert layer._nibble_weight_copy is None
    layer.nibble_copy_for_many_tokens = True
    got = layer(x)
    copy = layer._nibble_weight_copy
    assert copy is not None and copy.numel() == n * k // 2
    assert torch.equal(ops.unpack_lowbit(copy, 4, n * k), ops.unpack_lowbit(layer.packed_weight_indices, wbits, n * k))
    assert torch.equal(layer._nibble_weight_centroids[: 1 << wbits], layer._weight_codebook_centroids)
    assert torch.count_nonzero(layer._nibble_weight_centroids[1 << wbits:]) == 0
    # same operand values in the same K order: the sums agree bit for bit whenever both calls take the same
    # tile shape (the tile choice looks at the width); a K-split tile on one side only moves the last bit
    if not torch.equal(got, want):
        scale = want.float().abs().max().item()
        assert (got.float() - want.float()).abs().max().item() <= scale * 2.0 ** -7


def test_copy_is_opt_in(dev):
    """By default a 2- or 3-bit layer keeps its stored stream only: no second copy of the indices."""
    layer = make_layer(dev, 1024, 512, 3, 4)
    assert layer.nibble_copy_for_many_tokens is False
    layer(torch.randn(256, 1024, device=dev, dtype=torch.bfloat16))
    assert layer._nibble_weight_copy is None and layer._matmul_weight(4096)[1] == 3


def test_copy_follows_an_in_place_update(dev):
    """Indices written in place (same storage, version counter moved): the copy is rebuilt from them."""
    layer = make_layer(dev, 1024, 512, 3, 4)
    layer.nibble_copy_for_many_tokens = True
    other = make_layer(dev, 1024, 512, 3, 4, seed=9)
    many = torch.randn(256, 1024, device=dev, dtype=torch.bfloat16)
    first = layer(many)
    assert layer._nibble_weight_copy is not None
    with torch.no_grad():
        layer.packed_weight_indices.copy_(other.packed_weight_indices)
        layer.row_norms.copy_(other.row_norms)
        layer.bias.copy_(other.bias)
    second = layer(many)
    assert torch.equal(second, other(many)) and not torch.equal(second, first)
    assert layer._matmul_weight(256)[1] == 4   # and it is a copy of the new indices
    from orbitquant_amd import ops
    assert torch.equal(ops.unpack_lowbit(layer._nibble_weight_copy, 4, 512 * 1024),
                       ops.unpack_lowbit(other.packed_weight_indices, 3, 512 * 1024))


def test_copy_follows_the_weights(dev):
    layer = make_layer(dev, 1024, 512, 3, 4)
    layer.nibble_copy_for_many_tokens = True
    small, many = torch.randn(16, 1024, device=dev, dtype=torch.bfloat16), torch.randn(256, 1024, device=dev, dtype=torch.bfloat16)
    layer(small)
    assert layer._nibble_weight_copy is None                  # decode-sized calls read the stored stream
    assert layer._matmul_weight(64)[1] == 3 and layer._nibble_weight_copy is None
    first = layer(many)
    assert layer._nibble_weight_copy is not None and layer._matmul_weight(65)[1] == 4
    assert "_nibble_weight_copy" not in layer.state_dict()
    # other weights loaded into the same module: the copy is dropped and rebuilt from them
    other = make_layer(dev, 1024, 512, 3, 4, seed=9)
    layer.load_state_dict(other.state_dict(), strict=True)
    assert layer._nibble_weight_copy is None
    second = layer(many)
    assert torch.equal(second, other(many)) and not torch.equal(second, first)
    # a move drops the copy (it is rebuilt where the weights then are); widths without a copy never make one
    layer.cpu()
    assert layer._nibble_weight_copy is None and layer._matmul_weight(4096)[1] == 3
    layer.to(dev)
    assert torch.equal(layer(many), second) and layer._nibble_weight_centroids.dtype == torch.float32
    four = make_layer(dev, 1024, 512, 4, 4)
    four.nibble_copy_for_many_tokens = True
    four(many)
    assert four._nibble_weight_copy is None and four._matmul_weight(4096)[1] == 4
    six = make_layer(dev, 512, 64, 6, 6)
    six.nibble_copy_for_many_tokens = True
    six(torch.randn(300, 512, device=dev, dtype=torch.bfloat16))
    assert six._nibble_weight_copy is None


def test_prepared_copy_under_compile(dev):
    layer = make_layer(dev, 1024, 256, 3, 3)
    layer.nibble_copy_for_many_tokens = True
    x = torch.randn(384, 1024, device=dev, dtype=torch.bfloat16)
    want = layer(x)                      # builds the copy
    compiled = torch.compile(layer, fullgraph=True)
    assert torch.equal(compiled(x), want)
    fresh = make_layer(dev, 1024, 256, 3, 3)
    fresh.nibble_copy_for_many_tokens = True
    compiled_fresh = torch.compile(fresh, fullgraph=True)
    out = compiled_fresh(x)              # no copy yet and none can be built while tracing: the stored stream
    assert torch.equal(out, want) or (out.float() - want.float()).abs().max().item() <= want.float().abs().max().item() * 2.0 ** -7
    fresh.prepare_many_token_weights()
    assert fresh._nibble_weight_copy is not None
