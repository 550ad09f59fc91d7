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


def test_layers_restored_from_the_reference_written_artifact_match_the_oracle():
    """tests/golden/artifact_tiny was written by the reference's save_orbitquant_artifact.  Loaded by this
    package's loader onto the GPU, every restored OrbitLinear gives, on the inputs stored beside the artifact,
    the oracle's result computed from the artifact's own files (codes of the restored layer's quantizer bit for
    bit, outputs within the error bound) - and with that the reference's own outputs; the AdaLN modules match
    their fp64 contract within the bf16 rounding of the output."""
    from safetensors.torch import load_file

    from orbitquant_amd import OrbitLinear, load_artifact, ops
    from oracle import oracle_c
    from test_adaln_and_artifacts import GOLDEN_ARTIFACT, FluxTransformer2DModel, golden_artifact_oracle_outputs

    dev = torch.device("cuda:0")
    model = FluxTransformer2DModel()
    manifest = load_artifact(model, GOLDEN_ARTIFACT, device=dev)
    modules = dict(model.named_modules())
    outputs = load_file(GOLDEN_ARTIFACT / "reference_outputs.safetensors")
    rots = load_file(GOLDEN_ARTIFACT / "orbitquant_rotations.safetensors")
    books = load_file(GOLDEN_ARTIFACT / "orbitquant_codebooks.safetensors")
    for name in manifest["quantized_modules"]:
        layer = modules[name]
        assert isinstance(layer, OrbitLinear) and layer.packed_weight_indices.device.type == "cuda"
        x = outputs[name + ".x"]
        y_ref = outputs[name + ".y"].numpy().astype(np.float64)
        want, s, r = golden_artifact_oracle_outputs(name, x.numpy())
        k = x.shape[1]
        # the restored layer's quantizer against the oracle on the artifact's sidecar tables: bit for bit
        perm = rots[f"dim{k}_seed0_block16.permutation"].numpy()
        signs = rots[f"dim{k}_seed0_block16.signs"].numpy()
        inv = np.float32(rots[f"dim{k}_seed0_block16.normalization"].reshape(-1)[0].item())
        want_codes, want_s = oracle_c.rotate_quantize(x.numpy(), perm, signs, books[f"dim{k}_bits4.boundaries"].numpy(), 16, 1e-10, inv)
        codes, _, norms = ops.rotate_quantize(x.to(dev), layer._rotation_permutation, layer._rotation_signs,
                                              layer._activation_codebook_boundaries, block_size=layer.rotation.block_size,
                                              eps=layer.activation_eps, inv_sqrt_block=layer.rotation.normalization, code_format="u8")
        assert np.array_equal(codes.cpu().numpy(), want_codes), name
        assert np.array_equal(norms.cpu().numpy().view(np.int32), want_s.view(np.int32)), name
        bound = 2e-2 * s[:, None].astype(np.float64) * r[None, :] / np.sqrt(k)
        got = layer(x.to(dev)).double().cpu().numpy()                 # fp32 in, fp32 out
        assert (np.abs(got - want) <= bound + 1e-7).all(), name
        assert float((got * want).sum() / (np.linalg.norm(got) * np.linalg.norm(want))) >= 0.9999, name
        assert (np.abs(got - y_ref) <= bound + 1e-6).all(), name       # ... and the reference's own module output
        got16 = layer(x.to(dev).to(torch.bfloat16))
        want16, s16, _ = golden_artifact_oracle_outputs(name, x.to(torch.bfloat16).float().numpy())
        bound16 = 2e-2 * s16[:, None].astype(np.float64) * r[None, :] / np.sqrt(k)
        err16 = np.abs(got16.double().cpu().numpy() - want16)
        assert (err16 <= bound16 + np.abs(want16) * 2.0 ** -8 + 1e-7).all(), name
    for name in manifest["adaln_modules"]:
        x = outputs[name + ".x"]                                        # bf16-representable
        want, _, _ = golden_artifact_oracle_outputs(name, x.numpy())
        got = modules[name](x.to(dev)).double().cpu().numpy()
        # fp32 accumulation of exact bf16 products, then one rounding to bf16 (the bound of the AdaLN kernel's own test)
        k = x.shape[1]
        zero, _, _ = golden_artifact_oracle_outputs(name, np.zeros((1, k), np.float32))           # the bias
        weights, _, _ = golden_artifact_oracle_outputs(name, np.eye(k, dtype=np.float32))          # rows: W[:, j] + bias
        mass = np.abs(x.numpy().astype(np.float64)) @ np.abs(weights - zero) + np.abs(zero)
        # (the artifact holds an fp32 bias; the packed AdaLN kernel takes it as bf16, like the reference's kernels for it)
        tolerance = np.abs(want) * 2.0 ** -8 + np.abs(zero) * 2.0 ** -8 + mass * k * 2.0 ** -24 + 1e-30
        assert (np.abs(got - want) <= tolerance).all(), (name, float((np.abs(got - want) / tolerance).max()))
        y_ref = outputs[name + ".y"].numpy().astype(np.float64)
        assert np.abs(got - y_ref).max() <= 2.0 ** -7 * np.abs(want).max(), name
