"""MI355X-native quantized-linear forward for OrbitQuant models.

Public surface: `OrbitLinear`, `OrbitQuantConfig`, `recipe`, the host constants
(`get_rpbh_rotation`, `get_codebook`, `pack_lowbit`, `unpack_lowbit`,
`quantize_weight`) and `ops` (tensor wrappers over the C ABI).
"""

from .codebooks import LloydMaxCodebook, get_codebook
from .config import OrbitQuantConfig, recipe
from .packing import pack_lowbit, packed_length, unpack_lowbit
from .rotations import RPBHRotation, get_rpbh_rotation
from .weights import quantize_weight
from . import ops  # noqa: E402
from .layers import OrbitLinear  # noqa: E402

__all__ = [
    "LloydMaxCodebook", "OrbitLinear", "OrbitQuantConfig", "RPBHRotation", "get_codebook",
    "get_rpbh_rotation", "ops", "pack_lowbit", "packed_length", "quantize_weight", "recipe",
    "unpack_lowbit",
]
