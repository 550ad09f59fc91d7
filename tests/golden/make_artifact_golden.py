"""Writes tests/golden/artifact_tiny/: an artifact directory produced by the REFERENCE's own writer
(src/orbitquant/artifacts/writer.py: save_orbitquant_artifact) for a tiny mixed-bit model, plus
`reference_outputs.safetensors`: for every quantized module an fp32 input and the output of the
reference's module forward on it (CPU, its fp32/bf16 dequantized path).

Run once, in the build container only: it imports the reference package from the read-only
reference checkout (nothing of the reference is copied; what is committed is the data it wrote).
The loader in orbitquant_amd/artifacts.py is then tested against a layout it did not write itself.

    ORBITQUANT_KERNELS_AUTOFETCH=0 ORBITQUANT_DISABLE_CODEBOOK_DISK_CACHE=1 python tests/golden/make_artifact_golden.py

The model: three Flux-style blocks of width 64 (attention projections, a feed-forward pair, an AdaLN
modulation linear each) and an output projection; 2-bit weights with the reference's low-bit boundary
protection of one block, which gives the first and last block 4-bit weights (`module_bits` overrides),
4-bit activations, rotation blocks of 16.
"""

from __future__ import annotations

import json
import os
import shutil
import sys
from pathlib import Path

os.environ.setdefault("ORBITQUANT_KERNELS_AUTOFETCH", "0")
os.environ.setdefault("ORBITQUANT_DISABLE_CODEBOOK_DISK_CACHE", "1")
REFERENCE = Path(os.environ.get("OQ_REFERENCE_ROOT", "/root/reference"))
sys.path.insert(0, str(REFERENCE / "src"))

import torch  # noqa: E402
from safetensors.torch import save_file  # noqa: E402

DIM = 64


class FluxTransformer2DModel(torch.nn.Module):
    """Named like the class the reference's Flux policy looks for; three double-stream-like blocks."""

    def __init__(self):
        super().__init__()
        def block():
            return torch.nn.ModuleDict({
                "norm1": torch.nn.ModuleDict({"linear": torch.nn.Linear(DIM, 6 * DIM)}),
                "attn": torch.nn.ModuleDict({"to_q": torch.nn.Linear(DIM, DIM), "to_k": torch.nn.Linear(DIM, DIM),
                                             "to_v": torch.nn.Linear(DIM, DIM, bias=False),
                                             "to_out": torch.nn.ModuleList([torch.nn.Linear(DIM, DIM)])}),
                "ff": torch.nn.ModuleDict({"net": torch.nn.ModuleList([
                    torch.nn.ModuleDict({"proj": torch.nn.Linear(DIM, 2 * DIM)}), torch.nn.Identity(),
                    torch.nn.Linear(2 * DIM, DIM)])}),
            })
        self.transformer_blocks = torch.nn.ModuleList([block() for _ in range(3)])
        self.proj_out = torch.nn.Linear(DIM, DIM)


def main() -> int:
    from orbitquant.adaln import RTNInt4Linear
    from orbitquant.artifacts import save_orbitquant_artifact, validate_orbitquant_artifact
    from orbitquant.config import OrbitQuantConfig
    from orbitquant.layers import OrbitQuantLinear
    from orbitquant.modeling import quantize_linear_modules

    torch.manual_seed(1234)
    model = FluxTransformer2DModel()
    config = OrbitQuantConfig(weight_bits=2, activation_bits=4, block_size=16, lowbit_boundary_protection=1,
                              runtime_mode="dequant_bf16")
    summary = quantize_linear_modules(model, config)
    out = Path(__file__).resolve().parent / "artifact_tiny"
    if out.exists():
        shutil.rmtree(out)
    save_orbitquant_artifact(model, out, config=config, source_model_id="example/tiny-flux", source_revision="golden",
                             source_license="apache-2.0", summary=summary)
    report = validate_orbitquant_artifact(out)
    print("reference validator:", report if not hasattr(report, "ok") else report.ok)
    # the reference's own forward on a few rows, module by module (fp32 inputs, CPU)
    gen = torch.Generator().manual_seed(99)
    tensors = {}
    kinds = {}
    for name, module in model.named_modules():
        if isinstance(module, (OrbitQuantLinear, RTNInt4Linear)):
            x = torch.randn(5, module.in_features, generator=gen)
            x[1] *= 20.0
            x[2] = 0.0
            if isinstance(module, RTNInt4Linear):
                x = x.to(torch.bfloat16).float()
            with torch.no_grad():
                y = module(x)
            tensors[name + ".x"] = x.contiguous()
            tensors[name + ".y"] = y.float().contiguous()
            kinds[name] = type(module).__name__
    save_file(tensors, out / "reference_outputs.safetensors")
    (out / "reference_outputs.json").write_text(json.dumps({
        "modules": kinds, "quantized_modules": list(summary.quantized_modules), "adaln_modules": list(summary.adaln_modules),
        "note": "x: fp32 inputs; y: the reference module's forward(x) on CPU (runtime_mode dequant_bf16)"}, indent=1) + "\n")
    (out / "README.md").unlink()   # the generated model card: not read by any loader, not part of the fixture
    manifest = json.loads((out / "orbitquant_manifest.json").read_text())
    print("quantized:", len(manifest["quantized_modules"]), "adaln:", manifest["adaln_modules"], "module_bits:", manifest["module_bits"])
    print("wrote", out, sorted(p.name for p in out.iterdir()))
    return 0


if __name__ == "__main__":
    sys.exit(main())
