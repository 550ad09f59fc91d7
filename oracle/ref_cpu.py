"""Loader for oracle/_ref/liboq_ref_cpu.so: the reference's own CPU kernels for this
path (compiled by oracle/build.py from the reference checkout), registered as
`torch.ops.oq_ref_cpu.*` by oracle/ref_cpu_bind.cpp.  TEST INFRASTRUCTURE ONLY.

The two wrappers prepare arguments the way the reference's Python wrapper does
(native-kernels/orbitquant-packed-matmul/torch-ext/orbitquant_packed_matmul/__init__.py:66-160):
contiguous 2-D views, fp32 row norms / centroids / bias on the CPU, a dummy bias
with has_bias=False when there is none, caller-allocated output.
"""

from __future__ import annotations

from pathlib import Path

import torch

REF_SO = Path(__file__).resolve().parent / "_ref" / "liboq_ref_cpu.so"
_loaded = False


def available() -> bool:
    return REF_SO.exists()


def _ops():
    global _loaded
    if not _loaded:
        if not REF_SO.exists():
            raise RuntimeError(f"{REF_SO} is not built (run oracle/build.py where the reference checkout is present)")
        torch.ops.load_library(str(REF_SO))
        _loaded = True
    return torch.ops.oq_ref_cpu


def quantize_activations_cpu(x, permutation, signs, centroids, boundaries, *, eps, inv_sqrt_block, block_size):
    """-> centroid[code] * ||x||, same shape and dtype as x (CPU tensors)."""
    dim = x.shape[-1]
    values = x.contiguous().reshape(-1, dim)
    out = torch.empty_like(values)
    _ops().quantize_activations_cpu(
        out, values, permutation.to(torch.int32).contiguous(), signs.to(torch.int8).contiguous(),
        centroids.float().contiguous(), boundaries.float().contiguous(), float(eps), float(inv_sqrt_block),
        int(block_size))
    return out.reshape(x.shape)


def matmul_packed_weight(x, packed_weight_indices, row_norms, centroids, *, bits, out_features, in_features,
                         bias=None):
    x2 = x.contiguous().reshape(-1, in_features)
    out = torch.empty((x2.shape[0], out_features), dtype=x.dtype)
    if bias is None:
        bias_values, has_bias = torch.empty((1,), dtype=torch.float32), False
    else:
        bias_values, has_bias = bias.float().contiguous(), True
    _ops().matmul_packed_weight(
        out, x2, packed_weight_indices.to(torch.uint8).contiguous(), row_norms.float().contiguous(),
        centroids.float().contiguous(), bias_values, has_bias, int(bits), int(out_features), int(in_features),
        64, 64, 128)
    return out.reshape(*x.shape[:-1], out_features)
