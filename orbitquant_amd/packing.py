"""Low-bit index wire format (host side).

Value `i` of a flat index array occupies bits `[i*b, i*b + b)` of one
little-endian bit stream: bit `j` of the stream is bit `j % 8` of byte `j // 8`.
3- and 6-bit values may straddle bytes; the stream is `ceil(count*b/8)` bytes
(src/orbitquant/packing/bitpack.py:8-46,63-97; src/orbitquant/layers.py:84-85).
The packed GEMM/GEMV kernels decode this format directly from HBM.
"""

from __future__ import annotations

import numpy as np
import torch


def packed_length(value_count: int, bits: int) -> int:
    return (value_count * bits + 7) // 8


def _check_bits(bits: int) -> None:
    if bits <= 0 or bits > 8:
        raise ValueError("bits must be in [1, 8]")


def pack_lowbit(values: torch.Tensor, bits: int, *, validate: bool = True) -> torch.Tensor:
    _check_bits(bits)
    flat = values.detach().to(device="cpu").flatten()
    if validate and flat.numel() and (int(flat.min()) < 0 or int(flat.max()) >= (1 << bits)):
        raise ValueError(f"all values must fit in {bits} bits")
    as_bytes = flat.to(torch.uint8).numpy()
    bit_rows = np.unpackbits(as_bytes[:, None], axis=1, bitorder="little")[:, :bits]
    stream = np.packbits(bit_rows.reshape(-1), bitorder="little")
    return torch.from_numpy(stream.copy())


def unpack_lowbit(packed: torch.Tensor, bits: int, length: int) -> torch.Tensor:
    _check_bits(bits)
    if length < 0:
        raise ValueError("length must be non-negative")
    stream = packed.detach().to(device="cpu", dtype=torch.uint8).flatten().numpy()
    if stream.size < packed_length(length, bits):
        raise ValueError("packed buffer is shorter than length*bits")
    bit_stream = np.unpackbits(stream, bitorder="little")[: length * bits]
    bit_rows = np.zeros((length, 8), dtype=np.uint8)
    bit_rows[:, :bits] = bit_rows_view = bit_stream.reshape(length, bits)
    del bit_rows_view
    return torch.from_numpy(np.packbits(bit_rows, axis=1, bitorder="little").reshape(-1).copy())
