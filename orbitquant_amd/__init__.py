"""MI355X-native quantized-linear forward for OrbitQuant models.

Public surface: `OrbitLinear`, `OrbitLinearGroup`, `OrbitQuantConfig`, `recipe`, the host constants
(`get_rpbh_rotation`, `get_codebook`, `pack_lowbit`, `unpack_lowbit`,
`quantize_weight`), `RTNInt4Linear` (the AdaLN INT4 linear), `load_artifact` / `save_artifact`
(the reference's on-disk layout) and `ops` (tensor wrappers over the C ABI).
"""

from .codebooks import LloydMaxCodebook, get_codebook
from .config import OrbitQuantConfig, recipe
from .packing import pack_lowbit, packed_length, unpack_lowbit
from .rotations import RPBHRotation, get_rpbh_rotation
from .weights import quantize_weight
from . import ops  # noqa: E402
from .layers import OrbitLinear, OrbitLinearGroup  # noqa: E402
from .adaln import RTNInt4Linear, quantize_adaln_weight  # noqa: E402
from .artifacts import load_artifact, save_artifact  # noqa: E402

__all__ = [
    "LloydMaxCodebook", "OrbitLinear", "OrbitLinearGroup", "OrbitQuantConfig", "RPBHRotation", "RTNInt4Linear", "get_codebook",
    "get_rpbh_rotation", "load_artifact", "ops", "pack_lowbit", "packed_length", "quantize_adaln_weight",
    "quantize_weight", "recipe", "save_artifact", "unpack_lowbit",
]
