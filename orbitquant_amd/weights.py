"""Offline (host, torch) weight quantization: the tensors the packed GEMM reads.

Per output row (src/orbitquant/layers.py:121-125,201-215): `r = ||W_row||` in
fp32 on the unrotated row, `rotW = RPBH(W_row)`, `unit = rotW / max(r, eps)`,
`idx = #{j : boundaries[j] < unit}`, indices bit-packed as one flat little-endian
stream over the [N, K] index matrix, `row_norms = bf16(r)`.  A zero row keeps
`r = 0` and therefore dequantizes to exact zeros.

A weight that already sits on the GPU is quantized there (`oq_quantize_weight`, the
counterpart of the reference's device-side path, src/orbitquant/layers.py:102-125 with
src/orbitquant/kernels/triton_cuda.py:926-1039); a host weight takes the torch path below.
The two differ in one place only: the GPU kernel sums the squares of a row in the fixed order
of the activation kernel, the host path in torch's, so an index can differ where the last bit of
a norm moves a value across a boundary it sits on (the reference's own host and device paths
differ in the same way).
"""

from __future__ import annotations

import torch

from .codebooks import LloydMaxCodebook
from .packing import pack_lowbit
from .rotations import RPBHRotation


def quantize_weight_indices(
    weight: torch.Tensor,
    row_norms: torch.Tensor,
    *,
    rotation: RPBHRotation,
    codebook: LloydMaxCodebook,
    eps: float,
) -> torch.Tensor:
    rotated = rotation.apply_to_weight(weight)
    unit = rotated / row_norms.clamp_min(eps)[:, None]
    return codebook.quantize_indices(unit)


def quantize_weight(
    weight: torch.Tensor,
    *,
    rotation: RPBHRotation,
    codebook: LloydMaxCodebook,
    bits: int,
    eps: float,
    row_tile: int = 4096,
) -> tuple[torch.Tensor, torch.Tensor]:
    """-> (packed uint8 [ceil(N*K*bits/8)], row_norms bfloat16 [N]), on the GPU for a GPU weight the
    kernel takes, else on the CPU."""
    if weight.ndim != 2:
        raise ValueError("weight must be a matrix")
    n, k = weight.shape
    if (weight.device.type == "cuda" and k % 8 == 0 and k <= 16384 and 8 <= rotation.block_size <= 4096
            and weight.dtype in (torch.float32, torch.float16, torch.bfloat16)):
        from . import ops

        device = weight.device
        return ops.quantize_weight(
            weight, rotation.permutation.to(torch.int32).to(device), rotation.signs.to(torch.int8).to(device),
            codebook.boundaries.to(device), bits=bits, block_size=rotation.block_size, eps=eps,
            inv_sqrt_block=rotation.normalization, row_tile=row_tile)
    # Tiles must end on a byte boundary of the flat stream: rows * k * bits % 8 == 0.
    align = 8
    while (align // 2) * k * bits % 8 == 0 and align > 1:
        align //= 2
    row_tile = max(align, row_tile // align * align)
    pieces: list[torch.Tensor] = []
    norms = torch.empty(n, dtype=torch.bfloat16)
    for start in range(0, n, row_tile):
        tile = weight[start : start + row_tile].detach().to(device="cpu", dtype=torch.float32)
        r = tile.norm(dim=-1)
        idx = quantize_weight_indices(tile, r, rotation=rotation, codebook=codebook, eps=eps)
        pieces.append(pack_lowbit(idx, bits, validate=False))
        norms[start : start + row_tile] = r.to(torch.bfloat16)
    return torch.cat(pieces), norms
