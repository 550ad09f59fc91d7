"""GPU tests: the packed AdaLN INT4 linear against the oracle, and a model restored from an
artifact directory against the model it was saved from."""

from __future__ import annotations

import numpy as np
import pytest
import torch

from oracle import oracle_np as o

pytestmark = pytest.mark.gpu


def bf16(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(torch.bfloat16)


def adaln_case(M, N, K, group, with_bias, seed):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((N, K)) * 0.05).astype(np.float32)
    packed, scales, codes = o.adaln_quantize(w, group)
    x = bf16(rng.standard_normal((M, K)))
    bias = bf16(rng.standard_normal(N) * 0.1) if with_bias else None
    want = o.adaln_linear_f64(x.float().numpy(), codes, o.bf16_round(scales), None if bias is None else bias.float().numpy(), K, group)
    return x, torch.from_numpy(packed), bf16(scales), bias, w, want


@pytest.mark.parametrize("M,N,K,group,with_bias", [
    (1, 6912, 1152, 64, True),      # PixArt-scale modulation: 6 * hidden outputs, one token
    (2, 192, 1152, 64, False),
    (8, 100, 256, 64, True),        # N not a multiple of the 16 rows a wavefront owns
    (16, 64, 320, 64, True),
    (33, 70, 128, 32, True),        # three token blocks, the last ragged
    (3, 5, 70, 64, True),           # the reference's own shape: K not a multiple of the group -> padded stream
    (2, 7, 40, 16, False),
    (5, 9, 33, 64, True),           # odd K: the generic kernel
])
def test_adaln_int4_linear_against_the_oracle(M, N, K, group, with_bias):
    from orbitquant_amd import ops

    x, packed, scales, bias, _, want = adaln_case(M, N, K, group, with_bias, seed=M * 131 + N)
    dev = torch.device("cuda:0")
    got = ops.adaln_int4_linear(x.to(dev), packed.to(dev), scales.to(dev), bias=None if bias is None else bias.to(dev),
                                in_features=K, out_features=N, group_size=group)
    assert got.dtype == torch.bfloat16 and got.shape == (M, N)
    got = got.float().cpu().numpy().astype(np.float64)
    # fp32 accumulation of exact bf16 products, then one rounding to bf16:
    # |err| <= half a bf16 ulp of the result + K * 2^-24 * sum|x w| (a loose bound on the accumulation)
    weights = o.adaln_linear_f64(np.eye(K, dtype=np.float32), *_codes_scales(packed, scales, N, K, group), None, K, group).T
    mass = np.abs(x.float().numpy().astype(np.float64)) @ np.abs(weights).T + (0 if bias is None else np.abs(bias.float().numpy())[None, :])
    bound = np.abs(want) * 2.0 ** -8 + mass * K * 2.0 ** -24 + 1e-30
    assert (np.abs(got - want) <= bound).all(), float((np.abs(got - want) / bound).max())


def _codes_scales(packed, scales, N, K, group):
    groups = (K + group - 1) // group
    p = packed.numpy()
    codes = np.stack([p & 15, p >> 4], axis=-1).reshape(N, groups * group)
    return codes, scales.float().numpy().reshape(N, groups)


def test_adaln_module_and_packed_matmul_entry_agree():
    import orbitquant_packed_matmul as pm
    from orbitquant_amd import OrbitQuantConfig, RTNInt4Linear

    torch.manual_seed(3)
    dev = torch.device("cuda:0")
    linear = torch.nn.Linear(1152, 6 * 1152).to(dev)
    layer = RTNInt4Linear.from_linear(linear, config=OrbitQuantConfig())
    x = torch.randn(2, 1152, device=dev)
    y = layer(x)                                 # any float in -> bf16 arithmetic -> bf16 out, as the reference's module
    assert y.dtype == torch.bfloat16 and y.shape == (2, 6912)
    ref = torch.nn.functional.linear(x, linear.weight, linear.bias)
    assert torch.nn.functional.cosine_similarity(y.float().flatten(), ref.flatten(), dim=0) > 0.99   # 4-bit RTN of the weights
    direct = pm.matmul_packed_adaln_int4(x.to(torch.bfloat16), layer.packed_weight, layer.scales, bias=layer.bias,
                                         in_features=1152, out_features=6912, group_size=64)
    assert torch.equal(direct, y)
    # the host and device quantizers of the weight agree
    host = RTNInt4Linear.from_linear(linear.cpu(), config=OrbitQuantConfig())
    assert torch.equal(host.packed_weight, layer.packed_weight.cpu()) and torch.equal(host.scales, layer.scales.cpu())


def test_model_restored_from_an_artifact_computes_what_its_source_does(tmp_path):
    from orbitquant_amd import load_artifact, save_artifact
    from test_adaln_and_artifacts import Tiny, quantized_tiny

    model, config = quantized_tiny()
    save_artifact(model, tmp_path, config=config)
    dev = torch.device("cuda:0")
    restored = Tiny()
    load_artifact(restored, tmp_path, device=dev)
    model = model.to(dev)
    x = torch.randn(40, 16, device=dev)

    def run(net):
        h = x
        for block in net.blocks:
            mod = block.modulation(h[:1])
            shift, scale, gate = mod.chunk(3, dim=-1)
            a = block.norm(h) * (1 + scale) + shift
            h = h + gate * (block.attn["to_q"](a) + block.attn["to_v"](a))
            h = h + block.mlp(block.norm(h))
        return net.head(h)

    want, got = run(model), run(restored)
    assert torch.isfinite(want).all()
    head_same = torch.equal(model.head.weight.cpu(), restored.head.weight.cpu())
    assert head_same  # the unquantized tensors travel in model.safetensors too
    assert torch.equal(want, got)


@pytest.mark.parametrize("N,K,group,dtype", [
    (6912, 1152, 64, torch.float32), (37, 70, 64, torch.float32), (5, 40, 16, torch.bfloat16), (9, 300, 130, torch.float16),
])
def test_gpu_adaln_weight_quantizer_equals_the_oracle(N, K, group, dtype):
    from orbitquant_amd import ops

    rng = np.random.default_rng(N + K)
    w = torch.from_numpy((rng.standard_normal((N, K)) * 0.05).astype(np.float32)).to(dtype)
    w[0, :5] = torch.tensor([0.35, -0.35, 0.175, 0.125, 0.0]).to(dtype)   # exact ties when the group's absmax is 0.35
    w[0, 5:group] = 0
    if N > 3:
        w[3] = 0                                                           # all-zero groups: the scale floor
    packed, scales = ops.quantize_adaln_weight(w.to("cuda:0"), group_size=group)
    want_packed, want_scales, _ = o.adaln_quantize(w.float().numpy(), group)
    assert np.array_equal(scales.cpu().numpy(), want_scales)
    assert np.array_equal(packed.cpu().numpy(), want_packed)
