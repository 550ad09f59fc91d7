"""torch-tensor front end of the C ABI: allocation, dtype plumbing, stream.

The wrappers own allocation (as the reference's Python wrappers do,
native-kernels/orbitquant-packed-matmul/torch-ext/orbitquant_packed_matmul/__init__.py:130-160),
pass raw device pointers and the current HIP stream, and never synchronize.
"""

from __future__ import annotations

import torch

from . import _lib
from ._lib import (OQ_BF16, OQ_CODES_NIBBLE, OQ_CODES_U8, OQ_F16, OQ_F32, OQ_VALUES_NONE,
                   OQ_VALUES_SCALED, OQ_VALUES_UNIT_BF16)

_DTYPES = {torch.float32: OQ_F32, torch.float16: OQ_F16, torch.bfloat16: OQ_BF16}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DTYPES[t.dtype]
    except KeyError:
        raise ValueError(f"unsupported dtype {t.dtype}") from None


def _require_gpu(t: torch.Tensor, name: str) -> None:
    if t.device.type != "cuda":
        raise RuntimeError(f"{name} must live on an AMD GPU (torch device 'cuda'); got {t.device}")


def _operand(t: torch.Tensor | None, name: str, like: torch.Tensor, *, dtype=None, numel: int | None = None,
             min_numel: int | None = None) -> torch.Tensor | None:
    """An auxiliary tensor whose raw pointer goes to the library: it must sit on `like`'s
    device, have the expected dtype and element count, and is made contiguous."""
    if t is None:
        return None
    if t.device != like.device:
        raise ValueError(f"{name} is on {t.device}, the activations on {like.device}")
    if dtype is not None and t.dtype not in (dtype if isinstance(dtype, tuple) else (dtype,)):
        raise ValueError(f"{name} must be {dtype}, got {t.dtype}")
    if numel is not None and t.numel() != numel:
        raise ValueError(f"{name} must hold {numel} elements, got {t.numel()}")
    if min_numel is not None and t.numel() < min_numel:
        raise ValueError(f"{name} must hold at least {min_numel} elements, got {t.numel()}")
    return t if t.is_contiguous() else t.contiguous()


_FLOATS = (torch.float32, torch.float16, torch.bfloat16)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _workspace(nbytes: int, like: torch.Tensor) -> tuple[int | None, int, torch.Tensor | None]:
    """(address, size, tensor) of a workspace of `nbytes` for one call, from torch's caching allocator (the
    library allocates nothing: this wrapper owns allocation, as the reference's does).  The tensor is returned
    so that the caller keeps it alive until its call has been issued; stream-ordered reuse by the allocator
    makes it safe to drop then."""
    if nbytes <= 0:
        return None, 0, None
    buf = torch.empty(int(nbytes), dtype=torch.uint8, device=like.device)
    return buf.data_ptr(), int(nbytes), buf


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


class _OnDevice:
    """Make `t`'s device current for a launch; free when it already is (the usual case)."""

    __slots__ = ("_guard",)

    def __init__(self, t: torch.Tensor) -> None:
        index = t.device.index
        self._guard = None if index is None or index == torch.cuda.current_device() else torch.cuda.device(index)

    def __enter__(self):
        if self._guard is not None:
            self._guard.__enter__()

    def __exit__(self, *exc):
        if self._guard is not None:
            return self._guard.__exit__(*exc)
        return False


def rotate_plan(permutation: torch.Tensor, signs: torch.Tensor, boundaries: torch.Tensor, *, block_size: int,
                inv_sqrt_block: float) -> torch.Tensor:
    """The rotate plan of a layer (`oq_rotate_plan_build`): a uint8 blob on the constants' device
    that `rotate_quantize(plan=...)` and `quantized_linear(plan=...)` take to run the plan-based
    kernel.  Built by one small launch; valid for exactly these constants."""
    _require_gpu(permutation, "permutation")
    dim = permutation.numel()
    permutation = _operand(permutation, "permutation", permutation, dtype=torch.int32)
    signs = _operand(signs, "signs", permutation, dtype=torch.int8, numel=dim)
    boundaries = _operand(boundaries, "boundaries", permutation, dtype=torch.float32)
    lib = _lib.load()
    plan = torch.empty(int(lib.oq_rotate_plan_bytes(dim)), dtype=torch.uint8, device=permutation.device)
    with _OnDevice(permutation):
        rc = lib.oq_rotate_plan_build(permutation.data_ptr(), signs.data_ptr(), boundaries.data_ptr(),
                                      boundaries.numel() + 1, dim, int(block_size), float(inv_sqrt_block),
                                      plan.data_ptr(), _stream(permutation))
    _lib.check(rc, "oq_rotate_plan_build")
    plan._oq_plan_of = (int(dim), int(block_size), int(boundaries.numel() + 1))
    return plan


def quantize_weight(weight: torch.Tensor, permutation: torch.Tensor, signs: torch.Tensor, boundaries: torch.Tensor, *,
                    bits: int, block_size: int, eps: float, inv_sqrt_block: float,
                    row_tile: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """The weight side of a layer on the GPU (`oq_quantize_weight`): -> (packed uint8
    [ceil(N*K*bits/8)], row_norms bfloat16 [N]) on the weight's device.  `row_tile` bounds the
    rows converted per launch (the launches write disjoint byte ranges of the same stream, so the
    result does not depend on it; tiles end on byte boundaries because K is a multiple of 8)."""
    _require_gpu(weight, "weight")
    if weight.ndim != 2:
        raise ValueError("weight must be a matrix")
    n, k = weight.shape
    if weight.dtype not in _DTYPES:
        raise ValueError(f"unsupported weight dtype {weight.dtype}")
    w = weight.detach().contiguous()
    permutation = _operand(permutation, "permutation", w, dtype=torch.int32, numel=k)
    signs = _operand(signs, "signs", w, dtype=torch.int8, numel=k)
    boundaries = _operand(boundaries, "boundaries", w, dtype=torch.float32)
    plan = rotate_plan(permutation, signs, boundaries, block_size=block_size, inv_sqrt_block=inv_sqrt_block)
    packed = torch.empty((n * k * bits + 7) // 8, dtype=torch.uint8, device=w.device)
    norms = torch.empty(n, dtype=torch.bfloat16, device=w.device)
    lib = _lib.load()
    step = n if not row_tile else max(1, int(row_tile))
    with _OnDevice(w):
        for start in range(0, n, step):
            rows = min(step, n - start)
            rc = lib.oq_quantize_weight(
                w.data_ptr() + start * k * w.element_size(), _dt(w), rows, k, plan.data_ptr(), boundaries.data_ptr(),
                boundaries.numel() + 1, int(block_size), float(eps), float(inv_sqrt_block), int(bits),
                packed.data_ptr() + start * k * bits // 8, norms.data_ptr() + 2 * start, _stream(w))
            _lib.check(rc, "oq_quantize_weight")
    return packed, norms


def _plan_operand(plan: torch.Tensor | None, like: torch.Tensor, dim: int, block: int | None = None,
                  levels: int | None = None) -> torch.Tensor | None:
    """The plan as an operand.  Its byte count depends on the dimension alone, so a plan of another layer
    with the same dimension would pass that check: `rotate_plan` notes what a plan was built for on the
    tensor it returns, and a plan carrying such a note is refused here when block or levels differ.  (A
    plan without the note - a copy, a tensor the caller filled - is checked by the kernel, which stores
    NaN norms for a plan that does not match its launch.)"""
    if plan is None:
        return None
    expected = int(_lib.load().oq_rotate_plan_bytes(dim))
    made_for = getattr(plan, "_oq_plan_of", None)
    if made_for is not None:
        want = (int(dim), made_for[1] if block is None else int(block), made_for[2] if levels is None else int(levels))
        if tuple(made_for) != want:
            raise ValueError(f"this rotate plan was built for (dim, block, levels) = {tuple(made_for)}, the call has {want}")
    return _operand(plan, "plan", like, dtype=torch.uint8, numel=expected)


def rotate_quantize(
    x: torch.Tensor,
    permutation: torch.Tensor,
    signs: torch.Tensor,
    boundaries: torch.Tensor,
    *,
    block_size: int,
    eps: float,
    inv_sqrt_block: float,
    centroids: torch.Tensor | None = None,
    code_format: str | None = "u8",
    values: str | None = None,
    input_map: torch.Tensor | None = None,
    plan: torch.Tensor | None = None,
) -> tuple[torch.Tensor | None, torch.Tensor | None, torch.Tensor]:
    """-> (codes or None, values or None, norms[...]).

    plan: None, or `rotate_plan(...)` of the same permutation, signs, boundaries, block and
    factor: more than 16 rows then take the plan-based kernel (same results, much faster).

    input_map: None, or the table of an elementwise function f (`activation_table`): the
    result is that of rotate_quantize(f(x)), bit for bit, without f(x) ever being stored.

    code_format: "u8" ([..., K] uint8), "nibble" ([..., K/2] uint8) or None.
    values: None, "scaled" (centroid*norm in x.dtype) or "unit_bf16" (bf16 centroid).
    permutation int32, signs int8, boundaries/centroids fp32, all on x's device.
    """
    _require_gpu(x, "x")
    dim = x.shape[-1]
    rows = x.contiguous().reshape(-1, dim)
    m = rows.shape[0]
    lead = x.shape[:-1]
    levels = boundaries.numel() + 1
    permutation = _operand(permutation, "permutation", x, dtype=torch.int32, numel=dim)
    signs = _operand(signs, "signs", x, dtype=torch.int8, numel=dim)
    boundaries = _operand(boundaries, "boundaries", x, dtype=torch.float32)
    centroids = _operand(centroids, "centroids", x, dtype=torch.float32, numel=levels)
    codes = None
    fmt = OQ_CODES_U8
    if code_format == "u8":
        codes = torch.empty((m, dim), dtype=torch.uint8, device=x.device)
    elif code_format == "nibble":
        fmt = OQ_CODES_NIBBLE
        codes = torch.empty((m, dim // 2), dtype=torch.uint8, device=x.device)
    elif code_format is not None:
        raise ValueError(f"unknown code_format {code_format!r}")
    out_values = None
    mode = OQ_VALUES_NONE
    if values == "scaled":
        mode = OQ_VALUES_SCALED
        out_values = torch.empty_like(rows)
    elif values == "unit_bf16":
        mode = OQ_VALUES_UNIT_BF16
        out_values = torch.empty((m, dim), dtype=torch.bfloat16, device=x.device)
    elif values is not None:
        raise ValueError(f"unknown values mode {values!r}")
    if mode != OQ_VALUES_NONE and centroids is None:
        raise ValueError("centroids are required when values are requested")
    norms = torch.empty(m, dtype=torch.float32, device=x.device)
    if input_map is not None:
        if x.dtype not in (torch.float16, torch.bfloat16):
            raise ValueError("an input map needs float16 or bfloat16 inputs")
        if input_map.dtype != x.dtype or input_map.numel() != 65536 or input_map.device != x.device:
            raise ValueError("input_map must hold 65536 entries of x's dtype on x's device")
        input_map = input_map.contiguous()
    plan = _plan_operand(plan, x, dim, block_size, levels)
    lib = _lib.load()
    head = (m, dim, permutation.data_ptr(), signs.data_ptr(), boundaries.data_ptr(), _ptr(centroids), levels,
            int(block_size), float(eps), float(inv_sqrt_block))
    tail = (_ptr(codes), fmt, _ptr(out_values), mode, norms.data_ptr(), _stream(x))
    with _OnDevice(x):
        if input_map is None:
            rc = lib.oq_rotate_quantize(rows.data_ptr(), _dt(rows), *head, _ptr(plan), *tail)
        else:
            rc = lib.oq_rotate_quantize_mapped(rows.data_ptr(), _dt(rows), input_map.data_ptr(), *head, _ptr(plan), *tail)
    _lib.check(rc, "oq_rotate_quantize")
    if codes is not None:
        codes = codes.reshape(*lead, codes.shape[-1])
    if out_values is not None:
        out_values = out_values.reshape(*lead, dim)
    return codes, out_values, norms.reshape(lead)


def activation_table(fn, dtype: torch.dtype, device) -> torch.Tensor:
    """The table of an elementwise function for `rotate_quantize(input_map=...)`: fn applied
    to all 65536 values of a 16-bit dtype, in bit order, by the framework's own kernel for fn
    on `device`, so the fused path returns exactly what fn followed by the quantizer returns."""
    if dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("activation tables exist for float16 and bfloat16 only")
    bits = torch.arange(65536, dtype=torch.int32, device=device).to(torch.int16)
    out = fn(bits.view(dtype))
    if out.dtype != dtype or out.shape != bits.shape:
        raise ValueError("fn must be elementwise and keep the dtype")
    return out.contiguous()


def packed_linear(
    codes: torch.Tensor,
    token_norms: torch.Tensor,
    activation_centroids: torch.Tensor,
    packed_weight_indices: torch.Tensor,
    row_norms: torch.Tensor,
    weight_centroids: torch.Tensor,
    *,
    code_format: str,
    activation_bits: int,
    weight_bits: int,
    out_features: int,
    in_features: int,
    bias: torch.Tensor | None = None,
    output_dtype: torch.dtype = torch.bfloat16,
    output_map: torch.Tensor | None = None,
) -> torch.Tensor:
    _require_gpu(codes, "codes")
    fmt = {"u8": OQ_CODES_U8, "nibble": OQ_CODES_NIBBLE}[code_format]
    width = in_features if fmt == OQ_CODES_U8 else in_features // 2
    if codes.dtype != torch.uint8 or codes.shape[-1] != width:
        raise ValueError(f"codes must be uint8 with last dimension {width}")
    lead = codes.shape[:-1]
    flat = codes.contiguous().reshape(-1, width)
    m = flat.shape[0]
    expected = (out_features * in_features * weight_bits + 7) // 8
    packed_weight_indices = _operand(packed_weight_indices, "packed_weight_indices", codes, dtype=torch.uint8, min_numel=expected)
    row_norms = _operand(row_norms, "row_norms", codes, dtype=torch.bfloat16, numel=out_features)
    activation_centroids = _operand(activation_centroids, "activation_centroids", codes, dtype=torch.float32, numel=1 << activation_bits)
    weight_centroids = _operand(weight_centroids, "weight_centroids", codes, dtype=torch.float32, numel=1 << weight_bits)
    bias = _operand(bias, "bias", codes, dtype=_FLOATS, numel=out_features)
    out = torch.empty((m, out_features), dtype=output_dtype, device=codes.device)
    norms = _operand(token_norms.reshape(-1), "token_norms", codes, dtype=torch.float32, numel=m)
    if output_map is not None:
        if output_map.dtype != output_dtype or output_map.numel() != 65536 or output_map.device != codes.device \
                or output_dtype == torch.float32:
            raise ValueError("output_map must hold 65536 entries of the 16-bit output dtype on the codes' device")
        output_map = output_map.contiguous()
    lib = _lib.load()
    args = (flat.data_ptr(), fmt, norms.data_ptr(), activation_centroids.data_ptr(),
            int(activation_bits), packed_weight_indices.data_ptr(), int(weight_bits),
            row_norms.data_ptr(), weight_centroids.data_ptr(), _ptr(bias),
            _dt(bias) if bias is not None else OQ_F32, m, int(out_features), int(in_features),
            out.data_ptr(), _DTYPES[output_dtype])
    ws_ptr, ws_bytes, ws = _workspace(lib.oq_packed_linear_workspace_bytes(m, int(out_features), int(in_features), int(weight_bits),
                                                                            fmt, int(activation_bits)), codes)
    with _OnDevice(codes):
        if output_map is None:
            rc = lib.oq_packed_linear(*args, ws_ptr, ws_bytes, _stream(codes))
        else:
            rc = lib.oq_packed_linear_mapped(*args, output_map.data_ptr(), ws_ptr, ws_bytes, _stream(codes))
    del ws
    _lib.check(rc, "oq_packed_linear")
    return out.reshape(*lead, out_features)


def packed_linear_group(
    codes: torch.Tensor,
    token_norms: torch.Tensor,
    activation_centroids: torch.Tensor,
    weights,
    *,
    code_format: str,
    activation_bits: int,
    in_features: int,
    output_dtype: torch.dtype = torch.bfloat16,
) -> list[torch.Tensor]:
    """`packed_linear` of the same activation codes on several matrices, through one native call
    (one launch when the group is decode-sized, see oq_packed_linear_group).  `weights` is a sequence
    of (packed_weight_indices, row_norms, weight_centroids, weight_bits, out_features, bias or None);
    the biases present must share one dtype.  Returns the outputs in that order, each equal to what
    `packed_linear` returns for its matrix."""
    import ctypes

    _require_gpu(codes, "codes")
    fmt = {"u8": OQ_CODES_U8, "nibble": OQ_CODES_NIBBLE}[code_format]
    width = in_features if fmt == OQ_CODES_U8 else in_features // 2
    if codes.dtype != torch.uint8 or codes.shape[-1] != width:
        raise ValueError(f"codes must be uint8 with last dimension {width}")
    weights = list(weights)
    if not 1 <= len(weights) <= 64:
        raise ValueError("a group holds 1 to 64 matrices")
    lead = codes.shape[:-1]
    flat = codes.contiguous().reshape(-1, width)
    m = flat.shape[0]
    activation_centroids = _operand(activation_centroids, "activation_centroids", codes, dtype=torch.float32, numel=1 << activation_bits)
    norms = _operand(token_norms.reshape(-1), "token_norms", codes, dtype=torch.float32, numel=m)
    keep, outs, bias_dtype = [], [], None
    for packed, row_norms, cents, bits, n, bias in weights:
        expected = (n * in_features * bits + 7) // 8
        packed = _operand(packed, "packed_weight_indices", codes, dtype=torch.uint8, min_numel=expected)
        row_norms = _operand(row_norms, "row_norms", codes, dtype=torch.bfloat16, numel=n)
        cents = _operand(cents, "weight_centroids", codes, dtype=torch.float32, numel=1 << bits)
        bias = _operand(bias, "bias", codes, dtype=_FLOATS, numel=n)
        if bias is not None:
            if bias_dtype is not None and bias.dtype != bias_dtype:
                raise ValueError("the biases of a group must share one dtype")
            bias_dtype = bias.dtype
        keep.append((packed, row_norms, cents, int(bits), int(n), bias))
        outs.append(torch.empty((m, n), dtype=output_dtype, device=codes.device))
    count = len(keep)
    ptrs = ctypes.c_void_p * count
    lib = _lib.load()
    fmt_code = {"u8": OQ_CODES_U8, "nibble": OQ_CODES_NIBBLE}[code_format]
    ws_ptr, ws_bytes, ws = _workspace(max(lib.oq_packed_linear_workspace_bytes(m, k[4], int(in_features), k[3], fmt_code, int(activation_bits))
                                          for k in keep), codes)   # members run one after the other and share it
    with _OnDevice(codes):
        rc = lib.oq_packed_linear_group(
            flat.data_ptr(), fmt, norms.data_ptr(), activation_centroids.data_ptr(), int(activation_bits), count,
            ptrs(*[k[0].data_ptr() for k in keep]), (ctypes.c_int * count)(*[k[3] for k in keep]),
            ptrs(*[k[1].data_ptr() for k in keep]), ptrs(*[k[2].data_ptr() for k in keep]),
            ptrs(*[_ptr(k[5]) for k in keep]), _DTYPES[bias_dtype] if bias_dtype is not None else OQ_F32, m,
            (ctypes.c_int64 * count)(*[k[4] for k in keep]), int(in_features),
            ptrs(*[o.data_ptr() for o in outs]), _DTYPES[output_dtype], ws_ptr, ws_bytes, _stream(codes))
    del ws
    _lib.check(rc, "oq_packed_linear_group")
    return [o.reshape(*lead, o.shape[-1]) for o in outs]


def quantized_linear(
    x: torch.Tensor,
    permutation: torch.Tensor,
    signs: torch.Tensor,
    boundaries: torch.Tensor,
    act_centroids: torch.Tensor,
    packed_weight: torch.Tensor,
    row_norms: torch.Tensor,
    weight_centroids: torch.Tensor,
    *,
    block_size: int,
    eps: float,
    inv_sqrt_block: float,
    activation_bits: int,
    weight_bits: int,
    out_features: int,
    bias: torch.Tensor | None = None,
    input_map: torch.Tensor | None = None,
    output_map: torch.Tensor | None = None,
    plan: torch.Tensor | None = None,
) -> torch.Tensor:
    """rotate_quantize followed by packed_linear in one native call (same results): a single
    launch for one token of a 16-bit dtype (decode), two launches through scratch otherwise.
    input_map / output_map: tables (`activation_table`) of elementwise functions applied to the
    input before it is quantized / to the output before it is stored."""
    _require_gpu(x, "x")
    dim = x.shape[-1]
    rows = x.contiguous().reshape(-1, dim)
    m = rows.shape[0]
    permutation = _operand(permutation, "permutation", x, dtype=torch.int32, numel=dim)
    signs = _operand(signs, "signs", x, dtype=torch.int8, numel=dim)
    boundaries = _operand(boundaries, "boundaries", x, dtype=torch.float32, numel=(1 << activation_bits) - 1)
    act_centroids = _operand(act_centroids, "act_centroids", x, dtype=torch.float32, numel=1 << activation_bits)
    weight_centroids = _operand(weight_centroids, "weight_centroids", x, dtype=torch.float32, numel=1 << weight_bits)
    expected = (out_features * dim * weight_bits + 7) // 8
    packed_weight = _operand(packed_weight, "packed_weight", x, dtype=torch.uint8, numel=expected)
    row_norms = _operand(row_norms, "row_norms", x, dtype=torch.bfloat16, numel=out_features)
    if input_map is not None:
        if input_map.dtype != x.dtype or input_map.numel() != 65536 or input_map.device != x.device or x.dtype == torch.float32:
            raise ValueError("input_map must hold 65536 entries of x's 16-bit dtype on x's device")
        input_map = input_map.contiguous()
    if output_map is not None:
        if output_map.dtype != x.dtype or output_map.numel() != 65536 or output_map.device != x.device or x.dtype == torch.float32:
            raise ValueError("output_map must hold 65536 entries of the 16-bit output dtype on x's device")
        output_map = output_map.contiguous()
    bias = _operand(bias, "bias", x, dtype=_FLOATS, numel=out_features)
    plan = _plan_operand(plan, x, dim, block_size, 1 << activation_bits)
    nibble = activation_bits <= 4 and dim % 2 == 0
    codes = torch.empty((m, dim // 2 if nibble else dim), dtype=torch.uint8, device=x.device)
    norms = torch.empty(m, dtype=torch.float32, device=x.device)
    out = torch.empty((m, out_features), dtype=x.dtype, device=x.device)
    lib = _lib.load()
    ws_ptr, ws_bytes, ws = _workspace(lib.oq_packed_linear_workspace_bytes(
        m, int(out_features), dim, int(weight_bits), OQ_CODES_NIBBLE if nibble else OQ_CODES_U8, int(activation_bits)), x)
    with _OnDevice(x):
        rc = lib.oq_quantized_linear(
            rows.data_ptr(), _dt(rows), _ptr(input_map), m, dim, permutation.data_ptr(), signs.data_ptr(),
            boundaries.data_ptr(), act_centroids.data_ptr(), int(activation_bits), int(block_size), float(eps),
            float(inv_sqrt_block), _ptr(plan), packed_weight.data_ptr(), int(weight_bits), row_norms.data_ptr(),
            weight_centroids.data_ptr(), _ptr(bias), _dt(bias) if bias is not None else 0, out_features,
            codes.data_ptr(), norms.data_ptr(), out.data_ptr(), _dt(out), _ptr(output_map), ws_ptr, ws_bytes, _stream(x))
    del ws
    _lib.check(rc, "oq_quantized_linear")
    return out.reshape(*x.shape[:-1], out_features)


def quantized_linear_group(
    x: torch.Tensor,
    permutation: torch.Tensor,
    signs: torch.Tensor,
    boundaries: torch.Tensor,
    act_centroids: torch.Tensor,
    weights,
    *,
    block_size: int,
    eps: float,
    inv_sqrt_block: float,
    activation_bits: int,
    input_map: torch.Tensor | None = None,
    plan: torch.Tensor | None = None,
) -> list[torch.Tensor]:
    """`quantized_linear` of one input on several matrices in one native call: one quantization,
    then `packed_linear_group` (oq_quantized_linear_group).  `weights` as for
    `packed_linear_group`.  Every output equals `quantized_linear` on its matrix."""
    import ctypes

    _require_gpu(x, "x")
    dim = x.shape[-1]
    rows = x.contiguous().reshape(-1, dim)
    m = rows.shape[0]
    weights = list(weights)
    if not 1 <= len(weights) <= 64:
        raise ValueError("a group holds 1 to 64 matrices")
    permutation = _operand(permutation, "permutation", x, dtype=torch.int32, numel=dim)
    signs = _operand(signs, "signs", x, dtype=torch.int8, numel=dim)
    boundaries = _operand(boundaries, "boundaries", x, dtype=torch.float32, numel=(1 << activation_bits) - 1)
    act_centroids = _operand(act_centroids, "act_centroids", x, dtype=torch.float32, numel=1 << activation_bits)
    if input_map is not None:
        if input_map.dtype != x.dtype or input_map.numel() != 65536 or input_map.device != x.device or x.dtype == torch.float32:
            raise ValueError("input_map must hold 65536 entries of x's 16-bit dtype on x's device")
        input_map = input_map.contiguous()
    plan = _plan_operand(plan, x, dim, block_size, 1 << activation_bits)
    keep, outs, bias_dtype = [], [], None
    for packed, row_norms, cents, bits, n, bias in weights:
        expected = (n * dim * bits + 7) // 8
        packed = _operand(packed, "packed_weight_indices", x, dtype=torch.uint8, min_numel=expected)
        row_norms = _operand(row_norms, "row_norms", x, dtype=torch.bfloat16, numel=n)
        cents = _operand(cents, "weight_centroids", x, dtype=torch.float32, numel=1 << bits)
        bias = _operand(bias, "bias", x, dtype=_FLOATS, numel=n)
        if bias is not None:
            if bias_dtype is not None and bias.dtype != bias_dtype:
                raise ValueError("the biases of a group must share one dtype")
            bias_dtype = bias.dtype
        keep.append((packed, row_norms, cents, int(bits), int(n), bias))
        outs.append(torch.empty((m, n), dtype=x.dtype, device=x.device))
    nibble = activation_bits <= 4 and dim % 2 == 0
    codes = torch.empty((m, dim // 2 if nibble else dim), dtype=torch.uint8, device=x.device)
    norms = torch.empty(m, dtype=torch.float32, device=x.device)
    count = len(keep)
    ptrs = ctypes.c_void_p * count
    lib = _lib.load()
    ws_ptr, ws_bytes, ws = _workspace(max(lib.oq_packed_linear_workspace_bytes(
        m, k[4], dim, k[3], OQ_CODES_NIBBLE if nibble else OQ_CODES_U8, int(activation_bits)) for k in keep), x)
    with _OnDevice(x):
        rc = lib.oq_quantized_linear_group(
            rows.data_ptr(), _dt(rows), _ptr(input_map), m, dim, permutation.data_ptr(), signs.data_ptr(),
            boundaries.data_ptr(), act_centroids.data_ptr(), int(activation_bits), int(block_size), float(eps),
            float(inv_sqrt_block), _ptr(plan), count,
            ptrs(*[k[0].data_ptr() for k in keep]), (ctypes.c_int * count)(*[k[3] for k in keep]),
            ptrs(*[k[1].data_ptr() for k in keep]), ptrs(*[k[2].data_ptr() for k in keep]),
            ptrs(*[_ptr(k[5]) for k in keep]), _DTYPES[bias_dtype] if bias_dtype is not None else OQ_F32,
            (ctypes.c_int64 * count)(*[k[4] for k in keep]), codes.data_ptr(), norms.data_ptr(),
            ptrs(*[o.data_ptr() for o in outs]), _dt(x), ws_ptr, ws_bytes, _stream(x))
    del ws
    _lib.check(rc, "oq_quantized_linear_group")
    return [o.reshape(*x.shape[:-1], o.shape[-1]) for o in outs]


def matmul_packed_weight_values(
    x: torch.Tensor,
    packed_weight_indices: torch.Tensor,
    row_norms: torch.Tensor,
    weight_centroids: torch.Tensor,
    *,
    bits: int,
    out_features: int,
    in_features: int,
    bias: torch.Tensor | None = None,
    token_scale: torch.Tensor | None = None,
    output_dtype: torch.dtype | None = None,
) -> torch.Tensor:
    _require_gpu(x, "x")
    lead = x.shape[:-1]
    flat = x.contiguous().reshape(-1, in_features)
    m = flat.shape[0]
    out_dtype = x.dtype if output_dtype is None else output_dtype
    expected = (out_features * in_features * bits + 7) // 8
    packed_weight_indices = _operand(packed_weight_indices, "packed_weight_indices", x, dtype=torch.uint8, min_numel=expected)
    row_norms = _operand(row_norms, "row_norms", x, dtype=torch.bfloat16, numel=out_features)
    weight_centroids = _operand(weight_centroids, "weight_centroids", x, dtype=torch.float32, numel=1 << bits)
    bias = _operand(bias, "bias", x, dtype=_FLOATS, numel=out_features)
    token_scale = _operand(token_scale, "token_scale", x, dtype=torch.float32, numel=m)
    out = torch.empty((m, out_features), dtype=out_dtype, device=x.device)
    lib = _lib.load()
    ws_ptr, ws_bytes, ws = _workspace(lib.oq_matmul_packed_weight_workspace_bytes(m, int(out_features), int(in_features), int(bits),
                                                                                   _dt(x)), x)
    with _OnDevice(x):
        rc = lib.oq_matmul_packed_weight(
            flat.data_ptr(), _dt(flat), _ptr(token_scale), packed_weight_indices.data_ptr(), int(bits),
            row_norms.data_ptr(), weight_centroids.data_ptr(), _ptr(bias),
            _dt(bias) if bias is not None else OQ_F32, m, int(out_features), int(in_features),
            out.data_ptr(), _DTYPES[out_dtype], ws_ptr, ws_bytes, _stream(x))
    del ws
    _lib.check(rc, "oq_matmul_packed_weight")
    return out.reshape(*lead, out_features)


def adaln_int4_linear(x: torch.Tensor, packed_weight: torch.Tensor, scales: torch.Tensor, *, out_features: int,
                      in_features: int, group_size: int, bias: torch.Tensor | None = None) -> torch.Tensor:
    """The packed INT4 group-scaled linear of the AdaLN modules (`oq_matmul_packed_adaln_int4`):
    x is taken as bfloat16, the result is bfloat16 (as the reference's kernels for it)."""
    _require_gpu(x, "x")
    if x.shape[-1] != in_features:
        raise ValueError(f"expected input last dimension {in_features}, got {x.shape[-1]}")
    if group_size <= 0:
        raise ValueError("group_size must be positive")
    lead = x.shape[:-1]
    flat = x.to(torch.bfloat16).contiguous().reshape(-1, in_features)
    m = flat.shape[0]
    groups = (in_features + group_size - 1) // group_size
    packed_weight = _operand(packed_weight, "packed_weight", flat, dtype=torch.uint8,
                             numel=(out_features * groups * group_size * 4 + 7) // 8)
    scales = _operand(scales, "scales", flat, dtype=torch.bfloat16, numel=out_features * groups)
    if bias is not None and bias.dtype != torch.bfloat16:
        bias = bias.to(torch.bfloat16)
    bias = _operand(bias, "bias", flat, dtype=torch.bfloat16, numel=out_features)
    out = torch.empty((m, out_features), dtype=torch.bfloat16, device=flat.device)
    lib = _lib.load()
    with _OnDevice(flat):
        rc = lib.oq_matmul_packed_adaln_int4(flat.data_ptr(), packed_weight.data_ptr(), scales.data_ptr(), _ptr(bias), m,
                                             int(out_features), int(in_features), int(group_size), out.data_ptr(), _stream(flat))
    _lib.check(rc, "oq_matmul_packed_adaln_int4")
    return out.reshape(*lead, out_features)


def quantize_adaln_weight(weight: torch.Tensor, *, group_size: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Group-wise round-to-nearest INT4 of a weight on the GPU (`oq_quantize_adaln_weight`):
    -> (packed uint8 [N * groups * group_size / 2], scales float32 [N, groups])."""
    _require_gpu(weight, "weight")
    if weight.ndim != 2 or weight.dtype not in _DTYPES:
        raise ValueError("weight must be a float32/float16/bfloat16 matrix")
    if group_size <= 0 or group_size % 2:
        raise ValueError("the GPU quantizer takes even group sizes")
    weight = weight.contiguous()
    n, k = weight.shape
    groups = (k + group_size - 1) // group_size
    packed = torch.empty(n * groups * group_size // 2, dtype=torch.uint8, device=weight.device)
    scales = torch.empty(n, groups, dtype=torch.float32, device=weight.device)
    lib = _lib.load()
    with _OnDevice(weight):
        rc = lib.oq_quantize_adaln_weight(weight.data_ptr(), _DTYPES[weight.dtype], n, k, int(group_size), packed.data_ptr(),
                                          scales.data_ptr(), _stream(weight))
    _lib.check(rc, "oq_quantize_adaln_weight")
    return packed, scales


def pack_lowbit(values: torch.Tensor, bits: int) -> torch.Tensor:
    """uint8 indices -> the little-endian `bits`-wide stream (`oq_pack_lowbit`)."""
    _require_gpu(values, "values")
    values = _operand(values.reshape(-1), "values", values, dtype=torch.uint8)
    count = values.numel()
    packed = torch.empty((count * int(bits) + 7) // 8, dtype=torch.uint8, device=values.device)
    lib = _lib.load()
    with _OnDevice(values):
        rc = lib.oq_pack_lowbit(values.data_ptr(), int(bits), count, packed.data_ptr(), _stream(values))
    _lib.check(rc, "oq_pack_lowbit")
    return packed


def dequantize_packed_weight(packed_weight: torch.Tensor, row_norms: torch.Tensor, centroids: torch.Tensor, *, bits: int,
                             out_features: int, in_features: int, dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """centroids[index] * row_norm as a dense [out_features, in_features] matrix in the rotated
    basis (`oq_dequantize_packed_weight`)."""
    _require_gpu(packed_weight, "packed_weight")
    if dtype not in _DTYPES:
        raise ValueError(f"dtype must be one of {_FLOATS}")
    total = int(out_features) * int(in_features)
    packed_weight = _operand(packed_weight, "packed_weight", packed_weight, dtype=torch.uint8, min_numel=(total * int(bits) + 7) // 8)
    row_norms = _operand(row_norms, "row_norms", packed_weight, dtype=torch.bfloat16, numel=out_features)
    centroids = _operand(centroids, "centroids", packed_weight, dtype=torch.float32, numel=1 << int(bits))
    out = torch.empty(out_features, in_features, dtype=dtype, device=packed_weight.device)
    lib = _lib.load()
    with _OnDevice(packed_weight):
        rc = lib.oq_dequantize_packed_weight(packed_weight.data_ptr(), int(bits), row_norms.data_ptr(), centroids.data_ptr(),
                                             int(out_features), int(in_features), out.data_ptr(), _DTYPES[dtype], _stream(packed_weight))
    _lib.check(rc, "oq_dequantize_packed_weight")
    return out


def unpack_lowbit(packed: torch.Tensor, bits: int, length: int) -> torch.Tensor:
    _require_gpu(packed, "packed")
    packed = _operand(packed, "packed", packed, dtype=torch.uint8, min_numel=(int(length) * int(bits) + 7) // 8)
    out = torch.empty(length, dtype=torch.uint8, device=packed.device)
    lib = _lib.load()
    with _OnDevice(packed):
        rc = lib.oq_unpack_lowbit(packed.contiguous().data_ptr(), int(bits), int(length), out.data_ptr(),
                                  _stream(packed))
    _lib.check(rc, "oq_unpack_lowbit")
    return out
