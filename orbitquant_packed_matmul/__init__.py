"""`orbitquant_packed_matmul` for AMD Instinct MI355X (gfx950).

Same module name, function names, keyword arguments and return conventions as
the reference's native kernel package
(native-kernels/orbitquant-packed-matmul/torch-ext/orbitquant_packed_matmul/__init__.py:7-391),
so `orbitquant.kernels.native_packed_matmul` (which does a plain
`import orbitquant_packed_matmul` and probes functions by attribute,
src/orbitquant/kernels/native_packed_matmul.py:18-23,163-175) finds a GPU
backend on ROCm.  Every function launches hand-written HIP kernels through the
C ABI of `liborbitquant_hip.so`; there is no CPU implementation here, so the
CPU-only entry points of the reference package report themselves unavailable.

Differences from the reference wrappers, all widening:
  * `quantize_activations_packed_w4` / `quantize_activations_int8` accept any
    even input dimension up to 16384 and an optional `block_size` (the
    reference kernels are limited to a handful of dimensions and, for the
    packed form, to one block per row); fp32 inputs are accepted too.  The
    token scale divides (`x / (norm + eps)`, the Python reference's order)
    instead of multiplying by a reciprocal.
  * `threads`, `block_m/n/k`, `tile_m/n`, `async_packed` are accepted and
    ignored: tile selection is internal.  `weight_k_major=True` is rejected.
"""

from __future__ import annotations

import torch

from orbitquant_amd import _lib, ops

__all__ = [
    "matmul_packed_w4a4_int8",
    "matmul_packed_adaln_int4_cpu",
    "matmul_packed_weight",
    "quantize_activations_cpu",
    "quantize_activations_int8",
    "quantize_activations_packed_w4",
    "supports_cpu_activation",
    "supports_cpu_adaln",
    "supports_device",
]


def supports_device(device_type: str) -> bool:
    if device_type not in {"cpu", "cuda", "mps"}:
        raise ValueError(f"unknown device type {device_type!r}")
    if device_type != "cuda" or not getattr(torch.version, "hip", None):
        return False
    try:
        _lib.load()
    except Exception:
        return False
    return True


def supports_cpu_activation() -> bool:
    return False


def supports_cpu_adaln() -> bool:
    return False


def quantize_activations_cpu(*args, **kwargs):
    raise RuntimeError("this build of orbitquant_packed_matmul has no CPU kernels (AMD GPU only)")


def matmul_packed_adaln_int4_cpu(*args, **kwargs):
    raise RuntimeError("this build of orbitquant_packed_matmul has no CPU kernels (AMD GPU only)")


def matmul_packed_adaln_int4(x, packed_weight, scales, *, out_features, in_features, group_size, bias=None):
    """The AMD GPU form of `matmul_packed_adaln_int4_cpu` (same arguments and result, torch-ext
    `__init__.py`:163-204 of the reference): bf16 activations times the packed INT4 group-scaled
    weight, bf16 out."""
    from orbitquant_amd import ops

    if x.device.type != "cuda":
        raise RuntimeError("native packed AdaLN requires AMD GPU tensors (torch device 'cuda')")
    device = x.device
    return ops.adaln_int4_linear(
        x, packed_weight.to(device=device, dtype=torch.uint8), scales.to(device=device, dtype=torch.bfloat16),
        out_features=out_features, in_features=in_features, group_size=group_size,
        bias=None if bias is None else bias.to(device=device, dtype=torch.bfloat16))


def matmul_packed_weight(
    x: torch.Tensor,
    packed_weight_indices: torch.Tensor,
    row_norms: torch.Tensor,
    centroids: torch.Tensor,
    *,
    bits: int,
    out_features: int,
    in_features: int,
    bias: torch.Tensor | None = None,
    block_m: int = 64,
    block_n: int = 64,
    block_k: int = 128,
) -> torch.Tensor:
    if bits <= 0 or bits > 8:
        raise ValueError("bits must be in [1, 8]")
    if x.shape[-1] != in_features:
        raise ValueError(f"expected input last dimension {in_features}, got {x.shape[-1]}")
    if block_m <= 0 or block_n <= 0 or block_k <= 0:
        raise ValueError("packed matmul tile sizes must be positive")
    if not x.is_cuda:
        raise RuntimeError("this build of orbitquant_packed_matmul runs on AMD GPUs only")
    packed = packed_weight_indices.to(device=x.device, dtype=torch.uint8).contiguous()
    norms = row_norms.to(device=x.device, dtype=torch.bfloat16).contiguous()
    cents = centroids.to(device=x.device, dtype=torch.float32).contiguous()
    bias_values = None if bias is None else bias.to(device=x.device, dtype=x.dtype).contiguous()
    return ops.matmul_packed_weight_values(
        x, packed, norms, cents, bits=bits, out_features=out_features, in_features=in_features,
        bias=bias_values)


def _activation_inputs(x, permutation, signs, boundaries, block_size):
    if not x.is_cuda:
        raise RuntimeError("native activation quantization requires GPU tensors")
    if x.dtype not in {torch.float16, torch.bfloat16, torch.float32}:
        raise ValueError("x must be float16, bfloat16 or float32")
    dim = x.shape[-1]
    if permutation.numel() != dim or signs.numel() != dim:
        raise ValueError("permutation and signs must match the input dimension")
    if boundaries.numel() != 15:
        raise ValueError("boundaries must contain 15 values")
    block = dim if block_size is None else int(block_size)
    perm = permutation.to(device=x.device, dtype=torch.int32).contiguous()
    sgn = signs.to(device=x.device, dtype=torch.int8).contiguous()
    bnd = boundaries.to(device=x.device, dtype=torch.float32).contiguous()
    return perm, sgn, bnd, block


def quantize_activations_packed_w4(
    x: torch.Tensor,
    permutation: torch.Tensor,
    signs: torch.Tensor,
    boundaries: torch.Tensor,
    *,
    eps: float = 1e-12,
    inv_sqrt_block: float,
    threads: int = 256,
    block_size: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    if threads not in {128, 256, 512}:
        raise ValueError("threads must be 128, 256, or 512")
    perm, sgn, bnd, block = _activation_inputs(x, permutation, signs, boundaries, block_size)
    packed, _, norms = ops.rotate_quantize(
        x, perm, sgn, bnd, block_size=block, eps=eps, inv_sqrt_block=inv_sqrt_block, code_format="nibble")
    return packed, norms


def quantize_activations_int8(
    x: torch.Tensor,
    permutation: torch.Tensor,
    signs: torch.Tensor,
    boundaries: torch.Tensor,
    codes: torch.Tensor,
    *,
    eps: float = 1e-12,
    inv_sqrt_block: float,
    threads: int = 256,
    block_size: int | None = None,
) -> tuple[torch.Tensor, torch.Tensor]:
    if threads not in {128, 256, 512}:
        raise ValueError("threads must be 128, 256, or 512")
    if codes.numel() != 16:
        raise ValueError("codes must contain 16 values")
    perm, sgn, bnd, block = _activation_inputs(x, permutation, signs, boundaries, block_size)
    indices, _, norms = ops.rotate_quantize(
        x, perm, sgn, bnd, block_size=block, eps=eps, inv_sqrt_block=inv_sqrt_block, code_format="u8")
    table = codes.to(device=x.device, dtype=torch.int8)
    return table[indices.long()], norms


def matmul_packed_w4a4_int8(
    packed_activations: torch.Tensor,
    packed_weight_indices: torch.Tensor,
    token_norms: torch.Tensor,
    row_norms: torch.Tensor,
    activation_codes: torch.Tensor,
    weight_codes: torch.Tensor,
    *,
    activation_scale: float,
    weight_scale: float,
    out_features: int,
    in_features: int,
    bias: torch.Tensor | None = None,
    output_dtype: torch.dtype = torch.bfloat16,
    tile_m: int = 128,
    tile_n: int = 128,
    async_packed: bool = False,
    weight_k_major: bool = False,
) -> torch.Tensor:
    """out = (sum_k a_code[idx_a] * w_code[idx_w]) * s[m] * r[n] * (a_scale * w_scale) + bias.

    int8 code tables are exact in bf16 (|code| <= 127), so the bf16 matrix-core
    path reproduces the integer products exactly; accumulation is fp32.
    """
    if not packed_activations.is_cuda:
        raise RuntimeError("packed W4A4 matmul requires GPU tensors")
    if in_features <= 0 or in_features % 64 != 0:
        raise ValueError("in_features must be positive and divisible by 64")
    if packed_activations.shape[-1] != in_features // 2:
        raise ValueError(
            f"expected packed activation last dimension {in_features // 2}, got {packed_activations.shape[-1]}")
    if output_dtype not in {torch.float16, torch.bfloat16}:
        raise ValueError("output_dtype must be float16 or bfloat16")
    if (tile_m, tile_n) not in {(128, 128), (256, 128), (128, 256)}:
        raise ValueError("tile must be 128x128, 256x128, or 128x256")
    if weight_k_major:
        raise ValueError("weight_k_major layouts are not supported; pass the row-major packed stream")
    device = packed_activations.device
    scale = float(activation_scale) * float(weight_scale)
    norms = (token_norms.to(device=device, dtype=torch.float32) * scale).contiguous()
    return ops.packed_linear(
        packed_activations.to(torch.uint8), norms,
        activation_codes.to(device=device, dtype=torch.float32).contiguous(),
        packed_weight_indices.to(device=device, dtype=torch.uint8).contiguous(),
        row_norms.to(device=device, dtype=torch.bfloat16).contiguous(),
        weight_codes.to(device=device, dtype=torch.float32).contiguous(),
        code_format="nibble", activation_bits=4, weight_bits=4, out_features=out_features,
        in_features=in_features,
        bias=None if bias is None else bias.to(device=device, dtype=output_dtype).contiguous(),
        output_dtype=output_dtype)
