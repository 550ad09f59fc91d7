"""The configuration fields the quantized-linear forward reads.

Field names, defaults and validation follow the reference's `OrbitQuantConfig`
(src/orbitquant/config.py:60-186) for the subset this path consumes; `recipe`
mirrors src/orbitquant/recipes.py:7-33.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Any

SUPPORTED_BITS = (2, 3, 4, 6, 8)
RECIPES = {"w2a3": (2, 3), "w2a4": (2, 4), "w3a3": (3, 3), "w4a4": (4, 4), "w4a6": (4, 6)}


@dataclass
class OrbitQuantConfig:
    weight_bits: int = 4
    activation_bits: int = 4
    rotation_seed: int = 0
    block_size: int | str = "paper"
    codebook_version: int = 2
    activation_eps: float = 1e-10
    weight_row_tile_size: int = 256
    runtime_mode: str = "hip_packed"
    adaln_group_size: int = 64

    def __post_init__(self) -> None:
        if self.weight_bits not in SUPPORTED_BITS:
            raise ValueError(f"weight_bits must be one of {list(SUPPORTED_BITS)}")
        if self.activation_bits not in SUPPORTED_BITS:
            raise ValueError(f"activation_bits must be one of {list(SUPPORTED_BITS)}")
        if self.codebook_version != 2:
            raise ValueError("only codebook_version 2 is implemented")
        if self.block_size != "paper" and (not isinstance(self.block_size, int) or self.block_size <= 0):
            raise ValueError("block_size must be 'paper' or a positive int")
        if self.adaln_group_size <= 0:
            raise ValueError("adaln_group_size must be positive")
        if self.activation_eps <= 0:
            raise ValueError("activation_eps must be positive")
        if self.runtime_mode not in {"hip_packed", "auto_fused", "native_packed_matmul"}:
            raise ValueError("runtime_mode must be 'hip_packed' (aliases: auto_fused, native_packed_matmul)")


def recipe(name: str, **overrides: Any) -> OrbitQuantConfig:
    key = name.lower().replace("-", "")
    if key not in RECIPES:
        raise ValueError(f"unknown recipe {name!r}; choose one of {sorted(RECIPES)}")
    values: dict[str, Any] = {"weight_bits": RECIPES[key][0], "activation_bits": RECIPES[key][1]}
    values.update(overrides)
    return OrbitQuantConfig(**values)
