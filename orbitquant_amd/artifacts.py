"""Loading (and, for tests and small tools, writing) OrbitQuant artifact directories in the
reference's on-disk layout, so that a checkpoint quantized by the reference runs on this path
unchanged (src/orbitquant/artifacts/loader.py:54-116, writer.py:51-76, manifest.py:32-35,113):

    model.safetensors                   <module>.packed_weight_indices uint8 flat, <module>.row_norms bf16 [N],
                                        <module>.bias; AdaLN modules: <module>.packed_weight, <module>.scales, <module>.bias
    orbitquant_codebooks.safetensors    dim{K}_bits{b}.centroids | .boundaries            fp32
    orbitquant_rotations.safetensors    dim{K}_seed{s}_block{h}.permutation | .inverse_permutation | .signs | .normalization
    quantization_config.json            the quantization configuration (unknown fields are ignored here)
    orbitquant_manifest.json            quantized_modules, adaln_modules, module_bits (per-module weight widths), ...

`load_artifact` swaps every listed `nn.Linear` of a model for an `OrbitLinear` / `RTNInt4Linear`
skeleton (per-module widths from `module_bits`), checks the sidecar tensors against this
package's own generators (the reference's validator demands equality too,
src/orbitquant/artifacts/validator.py:192-202,275-281) and loads the state dict strictly.
"""

from __future__ import annotations

import dataclasses
import hashlib
import json
from pathlib import Path

import torch
from torch import nn

from .adaln import RTNInt4Linear
from .codebooks import get_codebook
from .config import OrbitQuantConfig
from .layers import OrbitLinear
from .rotations import get_rpbh_rotation

REQUIRED_FILES = ("model.safetensors", "orbitquant_codebooks.safetensors", "orbitquant_rotations.safetensors",
                  "quantization_config.json", "orbitquant_manifest.json")


def _get_module(model: nn.Module, name: str) -> nn.Module:
    module = model
    for part in name.split("."):
        if part.isdigit() and isinstance(module, (nn.ModuleList, nn.Sequential)):
            module = module[int(part)]
        elif isinstance(module, nn.ModuleDict):
            module = module[part]
        else:
            module = getattr(module, part)
    return module


def _set_module(model: nn.Module, name: str, replacement: nn.Module) -> None:
    parent_name, _, child = name.rpartition(".")
    parent = _get_module(model, parent_name) if parent_name else model
    if child.isdigit() and isinstance(parent, (nn.ModuleList, nn.Sequential)):
        parent[int(child)] = replacement
    elif isinstance(parent, nn.ModuleDict):
        parent[child] = replacement
    else:
        setattr(parent, child, replacement)


def config_from_dict(data: dict) -> OrbitQuantConfig:
    """The fields this path reads, out of the reference's full configuration record."""
    known = {f.name for f in dataclasses.fields(OrbitQuantConfig)}
    values = {k: v for k, v in data.items() if k in known}
    values.setdefault("codebook_version", 1)   # artifacts older than codebook versioning (config.py:206-208 of the reference)
    values["runtime_mode"] = "hip_packed"      # whatever back-end the artifact was made for, this package has one
    return OrbitQuantConfig(**values)


def _check_sidecars(path: Path, rotations: set, codebooks: set) -> None:
    from safetensors.torch import load_file

    problems: list[str] = []
    cb = load_file(path / "orbitquant_codebooks.safetensors")
    for dim, bits, version in sorted(codebooks):
        prefix = f"dim{dim}_bits{bits}"
        if f"{prefix}.centroids" not in cb or f"{prefix}.boundaries" not in cb:
            problems.append(f"{prefix}: missing from orbitquant_codebooks.safetensors")
            continue
        own = get_codebook(dim, bits, version)
        if not torch.equal(cb[f"{prefix}.centroids"], own.centroids) or not torch.equal(cb[f"{prefix}.boundaries"], own.boundaries):
            problems.append(f"{prefix}: the artifact's table differs from codebook version {version}")
    rot = load_file(path / "orbitquant_rotations.safetensors")
    for dim, seed, block in sorted(rotations):
        prefix = f"dim{dim}_seed{seed}_block{block}"
        if f"{prefix}.permutation" not in rot or f"{prefix}.signs" not in rot:
            problems.append(f"{prefix}: missing from orbitquant_rotations.safetensors")
            continue
        own = get_rpbh_rotation(dim, seed, block)
        if not torch.equal(rot[f"{prefix}.permutation"].to(torch.int64), own.permutation.to(torch.int64)):
            problems.append(f"{prefix}: permutation does not match the runtime rotation")
        if not torch.equal(rot[f"{prefix}.signs"].to(torch.int8), own.signs.to(torch.int8)):
            problems.append(f"{prefix}: signs do not match the runtime rotation")
    if problems:
        raise RuntimeError("artifact sidecar mismatch: " + "; ".join(problems))


def load_artifact(model: nn.Module, artifact_dir: str | Path, *, strict: bool = True, device: str | torch.device | None = None,
                  validate_checksums: bool = True, validate_sidecars: bool = True) -> dict:
    """Turn `model` (the unquantized architecture) into the quantized model stored in
    `artifact_dir`; returns the manifest.  With `device` the packed tensors are read straight
    onto that device and the swapped modules moved there."""
    from safetensors.torch import load_file

    path = Path(artifact_dir)
    missing = [name for name in REQUIRED_FILES if not (path / name).is_file()]
    if missing:
        raise RuntimeError(f"required artifact file missing: {missing}")
    config = config_from_dict(json.loads((path / "quantization_config.json").read_text(encoding="utf-8")))
    manifest = json.loads((path / "orbitquant_manifest.json").read_text(encoding="utf-8"))
    for field in ("weight_bits", "activation_bits"):
        if int(manifest[field]) != getattr(config, field):
            raise RuntimeError(f"artifact config/manifest mismatch: {field}")
    if validate_checksums:
        for name, want in manifest.get("checksums", {}).items():
            file = path / name
            if not file.is_file():
                raise RuntimeError(f"checksummed artifact file missing: {name}")
            if hashlib.sha256(file.read_bytes()).hexdigest() != want:
                raise RuntimeError(f"checksum mismatch: {name}")

    module_bits = {k: int(v) for k, v in manifest.get("module_bits", {}).items()}
    rotations, codebooks = set(), set()
    for name in manifest.get("quantized_modules", []):
        module = _get_module(model, name)
        if not isinstance(module, nn.Linear):
            raise TypeError(f"expected Linear at {name}, got {type(module).__name__}")
        bits = module_bits.get(name)
        module_config = config if bits is None or bits == config.weight_bits else dataclasses.replace(config, weight_bits=bits)
        replacement = OrbitLinear.empty_from_linear(module, config=module_config, module_name=name)
        rotations.add((replacement.in_features, config.rotation_seed, replacement.rotation.block_size))
        codebooks.add((replacement.in_features, module_config.weight_bits, config.codebook_version))
        codebooks.add((replacement.in_features, config.activation_bits, config.codebook_version))
        _set_module(model, name, replacement)
    for name in manifest.get("adaln_modules", []):
        module = _get_module(model, name)
        if not isinstance(module, nn.Linear):
            raise TypeError(f"expected Linear at {name}, got {type(module).__name__}")
        _set_module(model, name, RTNInt4Linear.empty_from_linear(module, config=config, module_name=name))
    if validate_sidecars:
        _check_sidecars(path, rotations, codebooks)

    target = None if device is None else torch.device(device)
    state = load_file(path / "model.safetensors", device=str(target) if target is not None and target.type == "cuda" else "cpu")
    missing_keys, unexpected = model.load_state_dict(state, strict=strict)
    if strict and (missing_keys or unexpected):
        raise RuntimeError(f"artifact state mismatch: missing={missing_keys}, unexpected={unexpected}")
    if target is not None:
        model.to(target)
    return manifest


def save_artifact(model: nn.Module, artifact_dir: str | Path, *, config: OrbitQuantConfig, source_model_id: str = "local",
                  source_revision: str = "unknown", source_license: str = "unknown") -> Path:
    """Write the quantized modules of `model` in the layout above (the five files this path
    consumes; the reference's writer adds a model card, prompts and benchmark records,
    src/orbitquant/artifacts/writer.py)."""
    from safetensors.torch import save_file

    path = Path(artifact_dir)
    path.mkdir(parents=True, exist_ok=True)
    quantized, adaln, bits_of, codebooks, rotations = [], [], {}, {}, {}
    for name, module in model.named_modules():
        if isinstance(module, OrbitLinear):
            quantized.append(name)
            if module.weight_bits != config.weight_bits:
                bits_of[name] = module.weight_bits
            for cb in (module.weight_codebook, module.activation_codebook):
                prefix = f"dim{cb.dim}_bits{cb.bits}"
                codebooks[f"{prefix}.centroids"] = cb.centroids.detach().cpu().contiguous()
                codebooks[f"{prefix}.boundaries"] = cb.boundaries.detach().cpu().contiguous()
            r = module.rotation
            prefix = f"dim{r.dim}_seed{r.seed}_block{r.block_size}"
            rotations[f"{prefix}.permutation"] = r.permutation.detach().cpu().contiguous()
            rotations[f"{prefix}.inverse_permutation"] = r.inverse_permutation.detach().cpu().contiguous()
            rotations[f"{prefix}.signs"] = r.signs.detach().cpu().contiguous()
            rotations[f"{prefix}.normalization"] = torch.tensor([r.normalization], dtype=torch.float32)
        elif isinstance(module, RTNInt4Linear):
            adaln.append(name)
    state = {k: v.detach().cpu().contiguous() for k, v in model.state_dict().items()}
    save_file(state, path / "model.safetensors")
    save_file(codebooks, path / "orbitquant_codebooks.safetensors")
    save_file(rotations, path / "orbitquant_rotations.safetensors")
    record = dataclasses.asdict(config)
    record.update(quant_method="orbitquant", rotation="rpbh", codebook="lloyd_max")
    (path / "quantization_config.json").write_text(json.dumps(record, indent=2, sort_keys=True) + "\n", encoding="utf-8")
    checksums = {name: hashlib.sha256((path / name).read_bytes()).hexdigest()
                 for name in ("model.safetensors", "orbitquant_codebooks.safetensors", "orbitquant_rotations.safetensors",
                              "quantization_config.json")}
    manifest = {
        "artifact_format": "orbitquant-v1", "source_model_id": source_model_id, "source_revision": source_revision,
        "source_license": source_license, "quant_method": "orbitquant", "weight_bits": config.weight_bits,
        "activation_bits": config.activation_bits, "rotation": "rpbh", "rotation_seed": config.rotation_seed,
        "block_size": config.block_size,
        "block_size_policy": "largest_power_of_two_dividing_dim" if config.block_size == "paper" else "explicit",
        "codebook": "lloyd_max", "codebook_version": config.codebook_version, "row_norm_dtype": "bfloat16",
        "runtime_mode": config.runtime_mode, "activation_eps": config.activation_eps,
        "adaln_group_size": config.adaln_group_size, "quantized_modules": quantized, "adaln_modules": adaln,
        "skipped_modules": [], "module_shapes": {k: list(v.shape) for k, v in state.items()},
        **({"module_bits": bits_of} if bits_of else {}), "checksums": checksums,
    }
    (path / "orbitquant_manifest.json").write_text(json.dumps(manifest, indent=2, sort_keys=True) + "\n", encoding="utf-8")
    return path
