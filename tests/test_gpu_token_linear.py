"""GPU tests of oq_quantized_linear: the whole layer forward in one native call, and its
single-launch form for one token.  The contract is bit identity with oq_rotate_quantize
followed by oq_packed_linear (both pinned to the oracle elsewhere)."""

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


def make_case(dev, m, k, n, wbits, abits, dtype, block, with_bias, seed):
    from orbitquant_amd.codebooks import get_codebook
    from orbitquant_amd.rotations import get_rpbh_rotation

    rot, acb, wcb = get_rpbh_rotation(k, 0, block), get_codebook(k, abits), get_codebook(k, wbits)
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, k, generator=g)
    x[torch.rand(m, k, generator=g) < 0.01] *= 20
    return dict(
        x=x.to(dtype).to(dev), perm=rot.permutation.to(torch.int32).to(dev), signs=rot.signs.to(torch.int8).to(dev),
        bounds=acb.boundaries.to(dev), cents=acb.centroids.to(dev), wcents=wcb.centroids.to(dev),
        packed=torch.randint(0, 256, ((n * k * wbits + 7) // 8,), generator=g, dtype=torch.uint8).to(dev),
        rn=(0.02 * (1 + 0.1 * torch.randn(n, generator=g))).to(torch.bfloat16).to(dev),
        bias=torch.randn(n, generator=g).to(dtype).to(dev) if with_bias else None,
        kw=dict(block_size=rot.block_size, eps=1e-10, inv_sqrt_block=rot.normalization), n=n, k=k, wbits=wbits, abits=abits)


def two_calls(c, input_map=None):
    from orbitquant_amd import ops

    fmt = "nibble" if c["abits"] <= 4 and c["k"] % 2 == 0 else "u8"
    codes, _, norms = ops.rotate_quantize(c["x"], c["perm"], c["signs"], c["bounds"], code_format=fmt,
                                          input_map=input_map, **c["kw"])
    return ops.packed_linear(codes, norms, c["cents"], c["packed"], c["rn"], c["wcents"], code_format=fmt,
                             activation_bits=c["abits"], weight_bits=c["wbits"], out_features=c["n"],
                             in_features=c["k"], bias=c["bias"], output_dtype=c["x"].dtype)


def one_call(c, input_map=None):
    from orbitquant_amd import ops

    return ops.quantized_linear(c["x"], c["perm"], c["signs"], c["bounds"], c["cents"], c["packed"], c["rn"],
                                c["wcents"], activation_bits=c["abits"], weight_bits=c["wbits"],
                                out_features=c["n"], bias=c["bias"], input_map=input_map, **c["kw"])


ONE_TOKEN = [
    # k, n, wbits, abits, dtype, block, bias       (all single-launch shapes: one token, K % 128 == 0, K <= 8192)
    (4096, 4096, 2, 4, torch.bfloat16, "paper", True),     # block 4096: three LDS stages
    (4096, 4096, 3, 4, torch.bfloat16, "paper", False),
    (4096, 14336, 4, 4, torch.bfloat16, "paper", True),    # four row groups per workgroup
    (4096, 6000, 3, 4, torch.float16, "paper", True),      # two row groups, N not a multiple of 32
    (1152, 4608, 4, 4, torch.bfloat16, "paper", True),     # block 128, single pass, padded to 2048
    (1024, 520, 4, 3, torch.bfloat16, 64, False),
    (2048, 1000, 3, 2, torch.float16, 512, True),
    (8192, 8192, 4, 4, torch.bfloat16, "paper", True),     # block 8192
    (6144, 3072, 2, 4, torch.bfloat16, "paper", True),     # block 2048, three passes
    (128, 16, 4, 4, torch.bfloat16, "paper", True),        # smallest
]


@pytest.mark.parametrize(("k", "n", "wbits", "abits", "dtype", "block", "with_bias"), ONE_TOKEN)
def test_one_token_single_launch_equals_two_launches(dev, k, n, wbits, abits, dtype, block, with_bias, library_switch):
    c = make_case(dev, 1, k, n, wbits, abits, dtype, block, with_bias, seed=k + n + wbits)
    want = two_calls(c)
    got = one_call(c)
    assert torch.equal(got, want)
    # and the switch that forces the two-launch route inside the same entry point
    library_switch("OQ_NO_TOKEN_LINEAR", "1")
    assert torch.equal(one_call(c), want)


def test_one_token_with_input_map(dev):
    from orbitquant_amd import ops

    gelu = torch.nn.functional.gelu
    for dtype in (torch.bfloat16, torch.float16):
        c = make_case(dev, 1, 4096, 4096, 3, 4, dtype, "paper", True, seed=3)
        table = ops.activation_table(gelu, dtype, dev)
        want = two_calls(dict(c, x=gelu(c["x"])))
        assert torch.equal(one_call(c, input_map=table), want)
        assert torch.equal(two_calls(c, input_map=table), want)


@pytest.mark.parametrize(("m", "k", "n", "wbits", "abits", "dtype"), [
    (2, 4096, 4096, 4, 4, torch.bfloat16),      # more than one token: streaming kernel, two launches
    (16, 1152, 4608, 4, 4, torch.bfloat16),
    (300, 1152, 4608, 4, 4, torch.bfloat16),    # tile kernel
    (1, 14336, 4096, 3, 4, torch.bfloat16),     # one token, row too long for the single launch
    (1, 4096, 4096, 6, 4, torch.bfloat16),      # weight width without a single-launch variant
    (1, 4096, 4096, 4, 6, torch.bfloat16),      # one code per byte
    (1, 1100, 96, 4, 4, torch.bfloat16),        # K % 128 != 0: generic kernel
    (5, 512, 256, 3, 3, torch.float32),         # fp32 inputs
])
def test_other_shapes_take_two_launches_with_the_same_result(dev, m, k, n, wbits, abits, dtype):
    c = make_case(dev, m, k, n, wbits, abits, dtype, "paper", True, seed=m + k)
    assert torch.equal(one_call(c), two_calls(c))


def test_quantized_linear_argument_checks(dev):
    from orbitquant_amd import _lib

    c = make_case(dev, 2, 512, 256, 4, 4, torch.bfloat16, "paper", False, seed=1)
    lib = _lib.load()
    out = torch.empty(2, 256, dtype=torch.bfloat16, device=dev)

    def call(m, codes, norms, a_bits=4):
        return lib.oq_quantized_linear(
            c["x"].data_ptr(), 2, None, m, 512, c["perm"].data_ptr(), c["signs"].data_ptr(), c["bounds"].data_ptr(),
            c["cents"].data_ptr(), a_bits, c["kw"]["block_size"], 1e-10, c["kw"]["inv_sqrt_block"], None,
            c["packed"].data_ptr(), 4, c["rn"].data_ptr(), c["wcents"].data_ptr(), None, 0, 256,
            codes, norms, out.data_ptr(), 2, None, None, 0, None)

    assert call(2, None, None) == 1 and b"scratch" in lib.oq_last_error()   # two tokens need the scratch buffers
    assert call(1, None, None) == 0                                           # one token does not
    assert call(2, None, None, a_bits=9) == 1
    assert call(0, None, None) == 0
    torch.cuda.synchronize()


def test_layer_forward_one_token_matches_batched_rows(dev):
    """A row computed alone (single launch) equals the same row computed in a batch (tile kernel inputs
    are the same codes; the matmul kernels differ, so this is a tolerance check, not bit identity)."""
    from orbitquant_amd import OrbitLinear, recipe

    torch.manual_seed(5)
    layer = OrbitLinear.from_linear(torch.nn.Linear(1024, 512), config=recipe("w4a4")).to(dev)
    x = torch.randn(40, 1024, dtype=torch.bfloat16, device=dev)
    batched = layer(x).float()
    single = torch.cat([layer(x[i : i + 1]) for i in range(40)]).float()
    scale = batched.abs().max().item()
    assert (batched - single).abs().max().item() <= 2e-2 * scale
    compiled = torch.compile(layer, fullgraph=True)
    assert torch.equal(compiled(x[:1]), layer(x[:1]))


@pytest.mark.parametrize("m", [1, 64])
def test_shared_input_quantization(dev, m, monkeypatch):
    """Layers marked `share_input_quantization` quantize a common input once; outputs equal the
    per-layer forward bit for bit; a changed or different input is quantized again."""
    from orbitquant_amd import OrbitLinear, OrbitQuantConfig, layers as layers_mod, ops

    torch.manual_seed(11)
    cfg = OrbitQuantConfig(weight_bits=4, activation_bits=4)
    q, k, v = (OrbitLinear.from_linear(torch.nn.Linear(1024, n), config=cfg).to(dev) for n in (1024, 512, 256))
    other = OrbitLinear.from_linear(torch.nn.Linear(2048, 256), config=cfg).to(dev)
    x = torch.randn(m, 1024, device=dev, dtype=torch.bfloat16)
    want = [layer(x) for layer in (q, k, v)]
    calls = []
    real = ops.rotate_quantize
    monkeypatch.setattr(layers_mod.ops, "rotate_quantize", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    for layer in (q, k, v, other):
        layer.share_input_quantization = True
    layers_mod._last_quantization.clear()
    got = [layer(x) for layer in (q, k, v)]
    assert len(calls) == 1
    assert all(torch.equal(a, b) for a, b in zip(got, want))
    other(torch.randn(m, 2048, device=dev, dtype=torch.bfloat16))   # another input in between: the entry is replaced
    assert torch.equal(k(x), want[1]) and len(calls) == 3
    x.add_(1)                                                        # same storage, new contents: the version counter moved
    fresh = k(x)
    assert len(calls) == 4 and not torch.equal(fresh, want[1])
    k.share_input_quantization = False
    assert torch.equal(k(x), fresh)
    y = x.clone()                                                    # same values, another tensor
    v(x)                                                             # still the entry k left
    assert len(calls) == 4
    v(y)
    assert len(calls) == 5
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                                    # another stream: not served from the entry
        before = len(calls)
        on_side = v(y)
        assert len(calls) == before + 1
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert torch.equal(on_side, v(y))


def test_shared_input_quantization_under_inference_mode(dev, monkeypatch):
    """Inference tensors have no version counter: such inputs are quantized by every layer (and the call
    does not raise); outputs equal the plain forward."""
    from orbitquant_amd import OrbitLinear, OrbitQuantConfig, layers as layers_mod, ops

    torch.manual_seed(12)
    cfg = OrbitQuantConfig(weight_bits=4, activation_bits=4)
    q, k = (OrbitLinear.from_linear(torch.nn.Linear(1024, n), config=cfg).to(dev) for n in (512, 256))
    calls = []
    real = ops.rotate_quantize
    monkeypatch.setattr(layers_mod.ops, "rotate_quantize", lambda *a, **kw: (calls.append(1), real(*a, **kw))[1])
    with torch.inference_mode():
        x = torch.randn(8, 1024, device=dev, dtype=torch.bfloat16)
        want = [layer(x) for layer in (q, k)]
        for layer in (q, k):
            layer.share_input_quantization = True
        layers_mod._last_quantization.clear()
        got = [layer(x) for layer in (q, k)]
    assert len(calls) == 2
    assert all(torch.equal(a, b) for a, b in zip(got, want))
