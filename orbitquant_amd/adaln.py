"""`RTNInt4Linear`: the symmetric INT4 round-to-nearest linear the reference uses for AdaLN
modulation weights (src/orbitquant/adaln.py:17-35,108-425), MI355X path.

Weight format (unchanged): every row is padded with zeros to whole groups of `group_size`
values; per group `scale = max(|w|, 1e-12) / 7` in fp32, `q = clamp(round(w / scale), -8, 7) + 8`
(round half to even), packed two per byte with the even value in the low nibble; scales are
stored as bfloat16 `[N, groups]`.  State dict keys: `packed_weight`, `scales`, `bias`
(src/orbitquant/transformers_ops.py:100-103).

Forward (bf16 in, bf16 out): `oq_matmul_packed_adaln_int4`, a stream over the packed weights
with the dequantized value `bf16((q - 8) * scale)` built in registers; no dequantized matrix
exists in memory and there is no CPU fallback.
"""

from __future__ import annotations

import torch
from torch import nn

from . import ops
from .config import OrbitQuantConfig
from .packing import pack_lowbit, packed_length


def quantize_adaln_weight(weight: torch.Tensor, *, group_size: int) -> tuple[torch.Tensor, torch.Tensor]:
    """-> (packed uint8 [N * groups * group_size / 2], scales float32 [N, groups])
    (src/orbitquant/adaln.py:17-35).  A weight on the GPU is quantized there by the library's
    kernel; a weight on the host by the torch operations below.  Both are IEEE fp32 and give the
    same bytes."""
    if weight.ndim != 2:
        raise ValueError("weight must be a matrix")
    if weight.device.type == "cuda" and group_size % 2 == 0 and weight.dtype in (torch.float32, torch.float16, torch.bfloat16):
        return ops.quantize_adaln_weight(weight, group_size=group_size)
    if weight.device.type == "cuda":   # odd group sizes: on the host, where torch's division is the IEEE one
        packed, scales = quantize_adaln_weight(weight.cpu(), group_size=group_size)
        return packed.to(weight.device), scales.to(weight.device)
    n, k = weight.shape
    groups = (k + group_size - 1) // group_size
    padded = torch.zeros(n, groups * group_size, dtype=torch.float32, device=weight.device)
    padded[:, :k] = weight.to(torch.float32)
    grouped = padded.reshape(n, groups, group_size)
    scales = grouped.abs().amax(dim=-1).clamp_min(1e-12) / 7.0
    signed = torch.round(grouped / scales[..., None]).clamp(-8, 7).to(torch.int16)
    packed = pack_lowbit((signed + 8).to(torch.uint8).flatten(), bits=4, validate=False)
    return packed.to(weight.device), scales


_LIB = torch.library.Library("orbitquant_amd", "FRAGMENT")
_LIB.define("adaln_int4_linear(Tensor x, Tensor packed_weight, Tensor scales, Tensor? bias, int out_features, "
            "int in_features, int group_size) -> Tensor")


def _adaln_forward(x, packed_weight, scales, bias, out_features, in_features, group_size):
    return ops.adaln_int4_linear(x, packed_weight, scales, out_features=out_features, in_features=in_features,
                                 group_size=group_size, bias=bias)


def _adaln_fake(x, packed_weight, scales, bias, out_features, in_features, group_size):
    return x.new_empty((*x.shape[:-1], out_features), dtype=torch.bfloat16)


_LIB.impl("adaln_int4_linear", _adaln_forward, "CUDA")
torch.library.register_fake("orbitquant_amd::adaln_int4_linear", _adaln_fake, lib=_LIB)


class RTNInt4Linear(nn.Module):
    def __init__(self, *, in_features: int, out_features: int, group_size: int, packed_weight: torch.Tensor,
                 scales: torch.Tensor, bias: torch.Tensor | None, module_name: str = "") -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.group_size = group_size
        self.module_name = module_name
        self.num_groups = (in_features + group_size - 1) // group_size
        expected = packed_length(out_features * self.num_groups * group_size, 4)
        if packed_weight.dtype != torch.uint8 or packed_weight.numel() != expected:
            raise ValueError(f"packed_weight must be uint8 with {expected} bytes")
        if scales.dtype != torch.bfloat16 or tuple(scales.shape) != (out_features, self.num_groups):
            raise ValueError("scales must be bfloat16 with shape (out_features, groups)")
        self.packed_weight = nn.Parameter(packed_weight.detach().flatten(), requires_grad=False)
        self.scales = nn.Parameter(scales.detach(), requires_grad=False)
        if bias is None:
            self.register_parameter("bias", None)
        else:
            self.bias = nn.Parameter(bias.detach().clone(), requires_grad=False)
        self.last_effective_runtime_mode: str | None = None

    @classmethod
    def from_weight(cls, weight: torch.Tensor, *, bias: torch.Tensor | None, config: OrbitQuantConfig,
                    module_name: str = "") -> "RTNInt4Linear":
        out_features, in_features = weight.shape
        packed, scales = quantize_adaln_weight(weight.detach(), group_size=config.adaln_group_size)
        return cls(in_features=in_features, out_features=out_features, group_size=config.adaln_group_size,
                   packed_weight=packed, scales=scales.to(torch.bfloat16), bias=None if bias is None else bias.detach(),
                   module_name=module_name)

    @classmethod
    def from_linear(cls, layer: nn.Linear, *, config: OrbitQuantConfig, module_name: str = "") -> "RTNInt4Linear":
        if not isinstance(layer, nn.Linear):
            raise TypeError(f"no OrbitQuant linear adapter registered for {type(layer).__name__}")
        return cls.from_weight(layer.weight.detach(), bias=layer.bias, config=config, module_name=module_name)

    @classmethod
    def empty_from_linear(cls, layer: nn.Linear, *, config: OrbitQuantConfig, module_name: str = "") -> "RTNInt4Linear":
        """A skeleton with the right tensor shapes for a state dict to be loaded into
        (src/orbitquant/adaln.py `empty_from_linear`)."""
        if not isinstance(layer, nn.Linear):
            raise TypeError(f"no OrbitQuant linear adapter registered for {type(layer).__name__}")
        n, k = layer.out_features, layer.in_features
        groups = (k + config.adaln_group_size - 1) // config.adaln_group_size
        device = layer.weight.device
        bias = None if layer.bias is None else torch.zeros(n, dtype=layer.bias.dtype, device=device)
        return cls(in_features=k, out_features=n, group_size=config.adaln_group_size,
                   packed_weight=torch.zeros(packed_length(n * groups * config.adaln_group_size, 4), dtype=torch.uint8, device=device),
                   scales=torch.zeros(n, groups, dtype=torch.bfloat16, device=device), bias=bias, module_name=module_name)

    def _apply(self, fn, recurse: bool = True):
        # A dtype cast of the model (`.half()`, `.float()`, `pipe.to(torch.float16)`) must not change the stored
        # format, and must not fail half-way either: the scales are put aside, moved with the rest, and come
        # back as the bfloat16 values they were (a cast to another dtype and back would round them).
        kept = self.scales.data
        result = super()._apply(fn, recurse=recurse)
        if self.scales.dtype != torch.bfloat16:
            self.scales.data = kept.to(device=self.scales.device)
        return result

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if x.shape[-1] != self.in_features:
            raise ValueError(f"expected last dimension {self.in_features}, got {x.shape[-1]}")
        if x.device.type != "cuda":
            raise RuntimeError("RTNInt4Linear runs on AMD GPUs only (torch device 'cuda'); there is no CPU fallback")
        self.last_effective_runtime_mode = "hip_packed_adaln_int4"
        return torch.ops.orbitquant_amd.adaln_int4_linear(x, self.packed_weight, self.scales, self.bias, self.out_features,
                                                          self.in_features, self.group_size)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, int4 group {self.group_size}"
