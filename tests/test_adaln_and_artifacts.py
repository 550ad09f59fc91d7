"""CPU tests: the oracle's AdaLN INT4 quantizer against hand-worked vectors and the properties
round-to-nearest fixes; the product's host quantizer against the oracle; and the artifact loader
(reference layout, per-module widths, strictness) on small models, without a GPU."""

from __future__ import annotations

import json

import numpy as np
import pytest
import torch

from oracle import oracle_np as o


# ---------------------------------------------------------------- AdaLN quantizer: oracle pins

def test_adaln_quantize_hand_worked_group():
    # absmax 7 -> scale exactly 1; ties round to even: 3.5 -> 4, 2.5 -> 2, -3.5 -> -4, 0.5 -> 0
    row = np.array([[7.0, -7.0, 3.5, 2.5, -3.5, 0.49, 0.5, -0.51]], dtype=np.float32)
    packed, scales, codes = o.adaln_quantize(row, group_size=8)
    assert scales.tolist() == [[1.0]]
    assert codes.tolist() == [[15, 1, 12, 10, 4, 8, 8, 7]]
    assert packed.tolist() == [0x1F, 0xAC, 0x84, 0x78]   # even index in the low nibble


def test_adaln_quantize_padding_zero_groups_and_error_bound():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((5, 70)).astype(np.float32)
    w[2] = 0
    packed, scales, codes = o.adaln_quantize(w, group_size=64)
    assert scales.shape == (5, 2) and codes.shape == (5, 128) and packed.size == 5 * 128 // 2
    assert (codes[:, 70:] == 8).all()                    # the zero padding quantizes to zero
    assert (codes[2] == 8).all() and np.allclose(scales[2], 1e-12 / 7)
    deq = (codes.astype(np.float32) - 8).reshape(5, 2, 64) * scales[..., None]
    err = np.abs(deq.reshape(5, 128)[:, :70] - w)
    assert (err <= np.repeat(scales, 64, axis=1)[:, :70] / 2 * (1 + 1e-6)).all()   # round to nearest
    hit = np.abs(codes.astype(int) - 8).reshape(5, 2, 64).max(axis=-1)
    assert (hit[[0, 1, 3, 4]] == 7).all()                # the largest value of a group maps to +-7
    # an independent reader of the nibble stream
    flat = np.array([(packed[i // 2] >> (4 * (i % 2))) & 15 for i in range(codes.size)], dtype=np.uint8)
    assert np.array_equal(flat, codes.reshape(-1))


def test_adaln_reference_test_vector():
    # tests/test_paper_reference_oracle.py:428-465 of the reference: 3 x 70 weights on a ramp, group 64
    w = torch.linspace(-1.5, 1.3, 210).reshape(3, 70).numpy()
    _, scales, codes = o.adaln_quantize(w, group_size=64)
    assert np.array_equal(scales[:, 0], (np.abs(w[:, :64]).max(axis=1) / np.float32(7)).astype(np.float32))
    assert codes[0, 0] == 1 and codes[2, 63] >= 8          # the most negative weight of row 0 -> -7; row 2 is positive at its end
    y = o.adaln_linear_f64(np.eye(70, dtype=np.float32)[:2], codes, o.bf16_round(scales), None, 70, 64)
    # a one-hot activation reads a column of the dequantized weight
    want = o.bf16_round((codes[:, :2].astype(np.float32) - 8) * o.bf16_round(scales)[:, :1])
    assert np.array_equal(y.T.astype(np.float32), want)


def test_product_adaln_quantizer_equals_the_oracle():
    from orbitquant_amd import quantize_adaln_weight

    rng = np.random.default_rng(1)
    for n, k, g in ((7, 70, 64), (16, 1152, 64), (3, 40, 16)):
        w = rng.standard_normal((n, k)).astype(np.float32) * 0.05
        w[0, :5] = [0.35, -0.35, 0.175, 0.125, 0.0]
        packed, scales = quantize_adaln_weight(torch.from_numpy(w), group_size=g)
        want_packed, want_scales, _ = o.adaln_quantize(w, g)
        assert np.array_equal(packed.numpy(), want_packed)
        assert np.array_equal(scales.numpy(), want_scales)


# ---------------------------------------------------------------- artifacts

class Block(torch.nn.Module):
    def __init__(self, dim):
        super().__init__()
        self.attn = torch.nn.ModuleDict({"to_q": torch.nn.Linear(dim, dim), "to_v": torch.nn.Linear(dim, dim, bias=False)})
        self.mlp = torch.nn.Sequential(torch.nn.Linear(dim, 2 * dim), torch.nn.GELU(), torch.nn.Linear(2 * dim, dim))
        self.modulation = torch.nn.Linear(dim, 3 * dim)
        self.norm = torch.nn.LayerNorm(dim)


class Tiny(torch.nn.Module):
    def __init__(self, dim=16):
        super().__init__()
        self.blocks = torch.nn.ModuleList([Block(dim), Block(dim)])
        self.head = torch.nn.Linear(dim, 4)


QUANTIZED = ["blocks.0.attn.to_q", "blocks.0.attn.to_v", "blocks.0.mlp.0", "blocks.0.mlp.2",
             "blocks.1.attn.to_q", "blocks.1.attn.to_v", "blocks.1.mlp.0", "blocks.1.mlp.2"]
BITS = {"blocks.0.attn.to_q": 4, "blocks.1.attn.to_v": 3}   # the others take the configuration's 2 bits


def quantized_tiny():
    import dataclasses

    from orbitquant_amd import OrbitLinear, OrbitQuantConfig, RTNInt4Linear
    from orbitquant_amd.artifacts import _get_module, _set_module

    torch.manual_seed(0)
    config = OrbitQuantConfig(weight_bits=2, activation_bits=4, block_size=8)
    model = Tiny()
    for name in QUANTIZED:
        cfg = dataclasses.replace(config, weight_bits=BITS.get(name, 2))
        _set_module(model, name, OrbitLinear.from_linear(_get_module(model, name), config=cfg, module_name=name))
    for name in ("blocks.0.modulation", "blocks.1.modulation"):
        _set_module(model, name, RTNInt4Linear.from_linear(_get_module(model, name), config=config, module_name=name))
    return model, config


def test_artifact_round_trip_is_strict_and_keeps_per_module_widths(tmp_path):
    from orbitquant_amd import OrbitLinear, RTNInt4Linear, load_artifact, save_artifact

    model, config = quantized_tiny()
    save_artifact(model, tmp_path, config=config)
    manifest = json.loads((tmp_path / "orbitquant_manifest.json").read_text())
    assert manifest["module_bits"] == BITS and manifest["quantized_modules"] == QUANTIZED
    restored = Tiny()
    out = load_artifact(restored, tmp_path)
    assert out["adaln_modules"] == ["blocks.0.modulation", "blocks.1.modulation"]
    assert isinstance(restored.blocks[0].attn["to_q"], OrbitLinear) and restored.blocks[0].attn["to_q"].weight_bits == 4
    assert restored.blocks[1].attn["to_v"].weight_bits == 3 and restored.blocks[1].mlp[0].weight_bits == 2
    assert isinstance(restored.blocks[1].modulation, RTNInt4Linear)
    assert isinstance(restored.head, torch.nn.Linear)          # not listed: untouched
    want, got = model.state_dict(), restored.state_dict()
    assert set(want) == set(got)
    for key in want:
        if "packed" in key or "row_norms" in key or "scales" in key:
            assert torch.equal(want[key], got[key]), key
    assert got["blocks.0.attn.to_q.packed_weight_indices"].numel() == 16 * 16 * 4 // 8
    assert got["blocks.1.attn.to_v.packed_weight_indices"].numel() == 16 * 16 * 3 // 8
    assert got["blocks.1.mlp.0.packed_weight_indices"].numel() == 32 * 16 * 2 // 8
    assert "blocks.0.attn.to_v.bias" not in got


def hand_written_artifact(path, model, config, *, extra_config=None, drop=None, add=None):
    """The five files as the reference's writer lays them out, built here from raw tensors (not
    through save_artifact), with the reference's full configuration record."""
    from safetensors.torch import save_file

    from orbitquant_amd import OrbitLinear

    state = {k: v.detach().clone().contiguous() for k, v in model.state_dict().items()}
    for key in drop or ():
        del state[key]
    state.update(add or {})
    save_file(state, path / "model.safetensors")
    codebooks, rotations = {}, {}
    for module in model.modules():
        if isinstance(module, OrbitLinear):
            for cb in (module.weight_codebook, module.activation_codebook):
                codebooks[f"dim{cb.dim}_bits{cb.bits}.centroids"] = cb.centroids.clone()
                codebooks[f"dim{cb.dim}_bits{cb.bits}.boundaries"] = cb.boundaries.clone()
            r = module.rotation
            prefix = f"dim{r.dim}_seed{r.seed}_block{r.block_size}"
            rotations[f"{prefix}.permutation"] = r.permutation.clone()
            rotations[f"{prefix}.inverse_permutation"] = r.inverse_permutation.clone()
            rotations[f"{prefix}.signs"] = r.signs.clone()
            rotations[f"{prefix}.normalization"] = torch.tensor([r.normalization], dtype=torch.float32)
    save_file(codebooks, path / "orbitquant_codebooks.safetensors")
    save_file(rotations, path / "orbitquant_rotations.safetensors")
    record = {  # every field of the reference's configuration (src/orbitquant/config.py of the reference)
        "quant_method": "orbitquant", "weight_bits": config.weight_bits, "activation_bits": config.activation_bits,
        "rotation": "rpbh", "rotation_seed": 0, "block_size": config.block_size, "codebook": "lloyd_max", "codebook_version": 2,
        "codebook_dtype": "float32", "row_norm_dtype": "bfloat16", "activation_norm_dtype": "float32", "weight_pack_dtype": "uint8",
        "adaln_policy": "int4_rtn", "adaln_group_size": 64, "runtime_mode": "auto_fused", "activation_kernel_backend": "auto",
        "activation_eps": 1e-10, "packed_matmul_block_m": 64, "packed_matmul_block_n": 64, "packed_matmul_block_k": 128,
        "packed_matmul_num_warps": 4, "weight_row_tile_size": 256, "target_policy": "auto", "modules_to_not_convert": [],
        "modules_dtype_dict": {}, "w4a4_int8_weight_cache": False, "lowbit_boundary_protection": "auto",
        "lowbit_protected_blocks": 4, "lowbit_protected_bits": 4, "lowbit_interior_protection": "auto"}
    record.update(extra_config or {})
    (path / "quantization_config.json").write_text(json.dumps(record))
    manifest = {"artifact_format": "orbitquant-v1", "source_model_id": "tiny", "source_revision": "0", "source_license": "mit",
                "weight_bits": config.weight_bits, "activation_bits": config.activation_bits, "rotation_seed": 0,
                "block_size": config.block_size, "codebook_version": 2, "quantized_modules": QUANTIZED,
                "adaln_modules": ["blocks.0.modulation", "blocks.1.modulation"], "skipped_modules": ["head"],
                "module_bits": BITS, "checksums": {}}
    (path / "orbitquant_manifest.json").write_text(json.dumps(manifest))


def test_loader_reads_the_reference_layout_and_ignores_fields_it_does_not_use(tmp_path):
    from orbitquant_amd import load_artifact

    model, config = quantized_tiny()
    hand_written_artifact(tmp_path, model, config)
    restored = Tiny()
    load_artifact(restored, tmp_path)
    for key, value in model.state_dict().items():
        assert torch.equal(value, restored.state_dict()[key]), key


def test_loader_strictness(tmp_path):
    from safetensors.torch import load_file, save_file

    from orbitquant_amd import load_artifact

    model, config = quantized_tiny()
    # a missing packed tensor, an unexpected tensor
    (tmp_path / "a").mkdir()
    hand_written_artifact(tmp_path / "a", model, config, drop=["blocks.1.mlp.2.row_norms"])
    with pytest.raises(RuntimeError, match="row_norms"):
        load_artifact(Tiny(), tmp_path / "a")
    (tmp_path / "b").mkdir()
    hand_written_artifact(tmp_path / "b", model, config, add={"blocks.0.attn.to_q.weight": torch.zeros(16, 16)})
    with pytest.raises(RuntimeError, match="to_q.weight"):
        load_artifact(Tiny(), tmp_path / "b")
    # the same two load when strict=False
    load_artifact(Tiny(), tmp_path / "a", strict=False)
    # a packed tensor of another width (module_bits says 4, the tensor holds 2 bits per index)
    (tmp_path / "c").mkdir()
    hand_written_artifact(tmp_path / "c", model, config,
                          add={"blocks.0.attn.to_q.packed_weight_indices": torch.zeros(16 * 16 * 2 // 8, dtype=torch.uint8)})
    with pytest.raises(RuntimeError, match="size mismatch"):
        load_artifact(Tiny(), tmp_path / "c")
    # a tampered sidecar, a missing file, a wrong module type, disagreeing config and manifest
    (tmp_path / "d").mkdir()
    hand_written_artifact(tmp_path / "d", model, config)
    rot = load_file(tmp_path / "d" / "orbitquant_rotations.safetensors")
    key = next(k for k in rot if k.endswith(".signs"))
    rot[key] = -rot[key]
    save_file(rot, tmp_path / "d" / "orbitquant_rotations.safetensors")
    with pytest.raises(RuntimeError, match="signs do not match"):
        load_artifact(Tiny(), tmp_path / "d")
    load_artifact(Tiny(), tmp_path / "d", validate_sidecars=False)
    (tmp_path / "d" / "orbitquant_codebooks.safetensors").unlink()
    with pytest.raises(RuntimeError, match="required artifact file missing"):
        load_artifact(Tiny(), tmp_path / "d")
    (tmp_path / "e").mkdir()
    hand_written_artifact(tmp_path / "e", model, config)
    broken = Tiny()
    broken.blocks[0].mlp[0] = torch.nn.Identity()
    with pytest.raises(TypeError, match="expected Linear at blocks.0.mlp.0"):
        load_artifact(broken, tmp_path / "e")
    (tmp_path / "f").mkdir()
    hand_written_artifact(tmp_path / "f", model, config, extra_config={"weight_bits": 3})
    with pytest.raises(RuntimeError, match="config/manifest mismatch"):
        load_artifact(Tiny(), tmp_path / "f")


def test_checksums_are_verified(tmp_path):
    from orbitquant_amd import load_artifact, save_artifact

    model, config = quantized_tiny()
    save_artifact(model, tmp_path, config=config)
    load_artifact(Tiny(), tmp_path)
    with open(tmp_path / "orbitquant_rotations.safetensors", "ab") as fh:
        fh.write(b"\0")
    with pytest.raises(RuntimeError, match="checksum mismatch"):
        load_artifact(Tiny(), tmp_path)


def test_adaln_module_survives_dtype_casts_of_the_model():
    """`model.half()` / `.float()` on a model that holds an RTNInt4Linear: no exception, nothing left
    half-converted; the scales stay the bfloat16 values they were, bias follows the cast like any parameter."""
    import torch
    from torch import nn

    from orbitquant_amd import OrbitQuantConfig, RTNInt4Linear

    torch.manual_seed(5)
    layer = RTNInt4Linear.from_linear(nn.Linear(130, 24), config=OrbitQuantConfig())
    model = nn.Sequential(nn.LayerNorm(130), layer)
    scales, packed = layer.scales.detach().clone(), layer.packed_weight.detach().clone()
    for cast in (model.half, model.float, lambda: model.to(torch.float16), model.bfloat16):
        cast()
        assert layer.scales.dtype == torch.bfloat16 and torch.equal(layer.scales, scales)
        assert layer.packed_weight.dtype == torch.uint8 and torch.equal(layer.packed_weight, packed)
    assert model[0].weight.dtype == torch.bfloat16 and layer.bias.dtype == torch.bfloat16


# ------------------------------------------------- an artifact the REFERENCE wrote (tests/golden/artifact_tiny)

GOLDEN_ARTIFACT = __import__("pathlib").Path(__file__).resolve().parent / "golden" / "artifact_tiny"


class FluxTransformer2DModel(torch.nn.Module):
    """The architecture tests/golden/make_artifact_golden.py quantized with the reference (same module names)."""

    def __init__(self, dim=64):
        super().__init__()

        def block():
            return torch.nn.ModuleDict({
                "norm1": torch.nn.ModuleDict({"linear": torch.nn.Linear(dim, 6 * dim)}),
                "attn": torch.nn.ModuleDict({"to_q": torch.nn.Linear(dim, dim), "to_k": torch.nn.Linear(dim, dim),
                                             "to_v": torch.nn.Linear(dim, dim, bias=False),
                                             "to_out": torch.nn.ModuleList([torch.nn.Linear(dim, dim)])}),
                "ff": torch.nn.ModuleDict({"net": torch.nn.ModuleList([
                    torch.nn.ModuleDict({"proj": torch.nn.Linear(dim, 2 * dim)}), torch.nn.Identity(),
                    torch.nn.Linear(2 * dim, dim)])}),
            })
        self.transformer_blocks = torch.nn.ModuleList([block() for _ in range(3)])
        self.proj_out = torch.nn.Linear(dim, dim)


def golden_artifact_oracle_outputs(name, x32):
    """fp64 output of quantized module `name` of the golden artifact on fp32 rows x32, computed by the oracle
    from the artifact's OWN files (state tensors, codebook and rotation sidecars, config, manifest):
    -> (want, token norms, row norms) for an OrbitLinear, (want, None, None) for an AdaLN module."""
    from safetensors.torch import load_file

    from oracle import oracle_c

    manifest = json.loads((GOLDEN_ARTIFACT / "orbitquant_manifest.json").read_text())
    config = json.loads((GOLDEN_ARTIFACT / "quantization_config.json").read_text())
    state = load_file(GOLDEN_ARTIFACT / "model.safetensors")
    bias = state.get(name + ".bias")
    bias = None if bias is None else bias.float().numpy()
    if name in manifest["adaln_modules"]:
        scales = state[name + ".scales"].float().numpy()
        n, groups = scales.shape
        g = int(config["adaln_group_size"])
        packed = state[name + ".packed_weight"].numpy()
        codes = np.stack([packed & 15, packed >> 4], axis=-1).reshape(n, groups * g)
        return o.adaln_linear_f64(x32, codes, scales, bias, x32.shape[1], g), None, None
    books = load_file(GOLDEN_ARTIFACT / "orbitquant_codebooks.safetensors")
    rots = load_file(GOLDEN_ARTIFACT / "orbitquant_rotations.safetensors")
    k = x32.shape[1]
    w_bits = int(manifest.get("module_bits", {}).get(name, manifest["weight_bits"]))
    a_bits = int(manifest["activation_bits"])
    rot = f"dim{k}_seed{config['rotation_seed']}_block{config['block_size']}"
    perm, signs = rots[rot + ".permutation"].numpy(), rots[rot + ".signs"].numpy()
    inv = np.float32(rots[rot + ".normalization"].reshape(-1)[0].item())
    ca, ba = books[f"dim{k}_bits{a_bits}.centroids"].numpy(), books[f"dim{k}_bits{a_bits}.boundaries"].numpy()
    cw = books[f"dim{k}_bits{w_bits}.centroids"].numpy()
    codes, s = oracle_c.rotate_quantize(x32, perm, signs, ba, int(config["block_size"]), float(config["activation_eps"]), inv)
    r = state[name + ".row_norms"].float().numpy()
    want = oracle_c.linear_from_codes(codes, s, ca, state[name + ".packed_weight_indices"].numpy(), w_bits, r, cw, bias, r.size)
    return want, s, r


def test_reference_written_artifact_loads_strictly():
    """The artifact directory was written by the reference's own save_orbitquant_artifact (a mixed-bit model:
    2-bit weights, first and last block protected at 4 bits, three AdaLN modules): this package's loader takes
    it as it is - checksums, sidecars equal to this package's generators, strict state dict."""
    import re

    from safetensors.torch import load_file

    from orbitquant_amd import OrbitLinear, RTNInt4Linear, load_artifact

    model = FluxTransformer2DModel()
    manifest = load_artifact(model, GOLDEN_ARTIFACT)
    assert manifest["artifact_format"] == "orbitquant-v1" and len(manifest["quantized_modules"]) == 18
    state = load_file(GOLDEN_ARTIFACT / "model.safetensors")
    got = model.state_dict()
    assert set(got) == set(state)
    for key, value in state.items():
        assert torch.equal(got[key].cpu(), value), key
    for name in manifest["quantized_modules"]:
        layer = dict(model.named_modules())[name]
        bits = manifest["module_bits"].get(name, 2)
        assert isinstance(layer, OrbitLinear) and layer.weight_bits == bits and layer.activation_bits == 4
        assert layer.rotation.block_size == 16
        assert state[name + ".packed_weight_indices"].numel() == layer.out_features * layer.in_features * bits // 8
        assert state[name + ".row_norms"].dtype == torch.bfloat16
    assert {manifest["module_bits"][n] for n in manifest["module_bits"]} == {4}
    assert sum(1 for n in manifest["quantized_modules"] if n not in manifest["module_bits"]) == 6   # the middle block: 2 bits
    for name in manifest["adaln_modules"]:
        assert isinstance(dict(model.named_modules())[name], RTNInt4Linear)
    assert isinstance(model.proj_out, torch.nn.Linear)   # skipped by the reference's policy: left alone
    # sidecar key names are what the reference's validator accepts (src/orbitquant/artifacts/validator.py:32-38)
    for key in load_file(GOLDEN_ARTIFACT / "orbitquant_codebooks.safetensors"):
        assert re.fullmatch(r"dim\d+_bits\d+\.(centroids|boundaries)", key), key
    for key in load_file(GOLDEN_ARTIFACT / "orbitquant_rotations.safetensors"):
        assert re.fullmatch(r"dim\d+_seed\d+_block\d+\.(permutation|inverse_permutation|signs|normalization)", key), key


def test_oracle_reads_the_reference_artifact_like_the_reference_does():
    """What the artifact's tensors MEAN: the oracle, fed only from the artifact's files, reproduces the outputs the
    reference's own modules gave on the same inputs (its CPU dequant_bf16 forward, stored beside the artifact)
    within the error bound of the path - so the loader's reading of the layout is pinned by the reference, not
    by this package's writer."""
    from safetensors.torch import load_file

    outputs = load_file(GOLDEN_ARTIFACT / "reference_outputs.safetensors")
    record = json.loads((GOLDEN_ARTIFACT / "reference_outputs.json").read_text())
    assert len(record["modules"]) == 21
    for name, kind in record["modules"].items():
        x, y = outputs[name + ".x"].numpy(), outputs[name + ".y"].numpy().astype(np.float64)
        want, s, r = golden_artifact_oracle_outputs(name, x)
        if kind == "RTNInt4Linear":
            # the reference's module rounds its output to bf16 (and accumulates in bf16-sized steps on some back-ends)
            assert np.abs(y - want).max() <= 2.0 ** -7 * np.abs(want).max(), name
            continue
        k = x.shape[1]
        bound = 2e-2 * s[:, None].astype(np.float64) * r[None, :] / np.sqrt(k)
        err = np.abs(y - want)
        assert (err <= bound + 1e-6).all(), (name, float((err / (bound + 1e-30)).max()))
        assert float((y * want).sum() / (np.linalg.norm(y) * np.linalg.norm(want))) >= 0.9999, name
        assert np.array_equal(y[2], want[2])   # the zero token: exactly the bias
