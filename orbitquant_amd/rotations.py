"""Randomized permuted block-Hadamard (RPBH) rotation constants and host apply.

The HIP rotate+quantize kernel consumes `permutation` (int32), `signs` (int8)
and `normalization`; this module draws them exactly as the reference does
(src/orbitquant/rotations/rpbh.py:55-72): one CPU `torch.Generator` seeded with
`seed`, `randperm(dim)` first, then `randint(0, 2, (dim,)) * 2 - 1` from the
same generator, `normalization = 1/sqrt(block)`.  `block_size="paper"` is the
largest power of two dividing `dim` (rpbh.py:13-18,36-38).

`apply_to_activations` is the host (torch) form used for offline weight
quantization and tests: gather by the permutation, multiply by the signs, one
unnormalized Walsh-Hadamard transform per block with butterfly distance
1, 2, 4, ... (src/orbitquant/rotations/fwht.py:19-25), then one multiply by
`normalization` (rpbh.py:80-84).
"""

from __future__ import annotations

import math
from functools import lru_cache

import torch


def is_power_of_two(value: int) -> bool:
    return value > 0 and value & (value - 1) == 0


def paper_block_size(dim: int) -> int:
    """Largest power of two that divides `dim`."""
    return dim & -dim


def fwht(x: torch.Tensor) -> torch.Tensor:
    """Unnormalized Walsh-Hadamard transform over the last dimension.

    Stage order is distance 1 first; every output of a stage is one add or one
    subtract of two outputs of the previous stage, so the result is
    bit-identical to any other schedule of the same butterflies.
    """
    n = x.shape[-1]
    if not is_power_of_two(n):
        raise ValueError("FWHT last dimension must be a power of two")
    lead = x.shape[:-1]
    y = x.contiguous().clone().reshape(-1, n)
    distance = 1
    while distance < n:
        pairs = y.view(-1, n // (2 * distance), 2, distance)
        top = pairs[:, :, 0, :] + pairs[:, :, 1, :]
        bottom = pairs[:, :, 0, :] - pairs[:, :, 1, :]
        y = torch.stack((top, bottom), dim=2).reshape(-1, n)
        distance *= 2
    return y.reshape(*lead, n)


class RPBHRotation:
    """`apply_to_activations(x)` computes x @ R for row vectors."""

    def __init__(self, dim: int, seed: int = 0, block_size: int | str = "paper") -> None:
        if dim <= 0:
            raise ValueError("dim must be positive")
        if block_size == "paper":
            block_size = paper_block_size(dim)
        if not isinstance(block_size, int):
            raise TypeError("block_size must be an int or 'paper'")
        if block_size <= 0:
            raise ValueError("block_size must be positive")
        if not is_power_of_two(block_size):
            raise ValueError("block_size must be a power of two")
        if dim % block_size != 0:
            raise ValueError("block_size must divide dim")
        generator = torch.Generator(device="cpu")
        generator.manual_seed(int(seed))
        permutation = torch.randperm(dim, generator=generator, dtype=torch.long, device="cpu")
        signs = torch.randint(0, 2, (dim,), generator=generator, dtype=torch.int8, device="cpu")
        inverse = torch.empty_like(permutation)
        inverse[permutation] = torch.arange(dim, dtype=torch.long)
        self.dim = dim
        self.seed = int(seed)
        self.block_size = block_size
        self.num_blocks = dim // block_size
        self.permutation = permutation
        self.inverse_permutation = inverse
        self.signs = signs * 2 - 1
        self.normalization = 1.0 / math.sqrt(block_size)

    def _check(self, x: torch.Tensor) -> None:
        if x.shape[-1] != self.dim:
            raise ValueError(f"expected last dimension {self.dim}, got {x.shape[-1]}")

    def apply_to_activations(self, x: torch.Tensor) -> torch.Tensor:
        self._check(x)
        gathered = x.index_select(-1, self.permutation.to(x.device))
        gathered = gathered * self.signs.to(device=x.device, dtype=x.dtype)
        blocks = gathered.reshape(*x.shape[:-1], self.num_blocks, self.block_size)
        return (fwht(blocks) * self.normalization).reshape(x.shape)

    def apply_to_weight(self, weight: torch.Tensor) -> torch.Tensor:
        if weight.ndim != 2:
            raise ValueError("weight must be a rank-2 tensor")
        return self.apply_to_activations(weight)

    def apply_inverse_to_activations(self, x: torch.Tensor) -> torch.Tensor:
        self._check(x)
        blocks = x.reshape(*x.shape[:-1], self.num_blocks, self.block_size)
        y = (fwht(blocks) * self.normalization).reshape(x.shape)
        y = y * self.signs.to(device=x.device, dtype=x.dtype)
        return y.index_select(-1, self.inverse_permutation.to(x.device))

    def apply_inverse_to_weight(self, weight: torch.Tensor) -> torch.Tensor:
        if weight.ndim != 2:
            raise ValueError("weight must be a rank-2 tensor")
        return self.apply_inverse_to_activations(weight)


@lru_cache(maxsize=256)
def get_rpbh_rotation(dim: int, seed: int = 0, block_size: int | str = "paper") -> RPBHRotation:
    return RPBHRotation(dim=dim, seed=seed, block_size=block_size)


def clear_rotation_cache() -> None:
    get_rpbh_rotation.cache_clear()
