"""ctypes binding of `liborbitquant_hip.so` (the C ABI in include/orbitquant_hip.h).

There is no CPU fallback: if the library is missing, or a call fails, an
exception is raised.
"""

from __future__ import annotations

import ctypes
import os
from pathlib import Path

LIB_PATH = Path(os.environ.get("ORBITQUANT_HIP_LIB") or Path(__file__).resolve().parent / "liborbitquant_hip.so")

OQ_F32, OQ_F16, OQ_BF16 = 0, 1, 2
OQ_CODES_U8, OQ_CODES_NIBBLE = 0, 1
OQ_VALUES_NONE, OQ_VALUES_SCALED, OQ_VALUES_UNIT_BF16 = 0, 1, 2

_STATUS = {1: "invalid argument", 2: "unsupported", 3: "launch failure"}

EXPORTS = (
    "oq_device_ok", "oq_last_error", "oq_version", "oq_debug_override", "oq_rotate_quantize", "oq_rotate_plan_bytes", "oq_rotate_plan_build", "oq_quantize_weight", "oq_rotate_quantize_mapped",
    "oq_packed_linear", "oq_packed_linear_group", "oq_packed_linear_mapped", "oq_quantized_linear", "oq_quantized_linear_group", "oq_quantized_linear_static", "oq_matmul_packed_weight", "oq_matmul_packed_adaln_int4", "oq_quantize_adaln_weight", "oq_unpack_lowbit", "oq_pack_lowbit",
    "oq_dequantize_packed_weight", "oq_packed_linear_workspace_bytes", "oq_matmul_packed_weight_workspace_bytes",
)

_lib = None


class OrbitQuantHipError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise OrbitQuantHipError(
            f"{LIB_PATH} is missing: build it with `python -m orbitquant_amd.build` "
            "(there is no CPU fallback for the quantized-linear forward)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    c_i64, c_int, c_f, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p
    lib.oq_last_error.restype = ctypes.c_char_p
    lib.oq_version.restype = ctypes.c_char_p
    lib.oq_device_ok.restype = c_int
    lib.oq_rotate_quantize.restype = c_int
    lib.oq_rotate_quantize.argtypes = [vp, c_int, c_i64, c_i64, vp, vp, vp, vp, c_int, c_i64, c_f, c_f, vp,
                                       vp, c_int, vp, c_int, vp, vp]
    lib.oq_rotate_plan_bytes.restype = ctypes.c_uint64
    lib.oq_rotate_plan_bytes.argtypes = [c_i64]
    lib.oq_rotate_plan_build.restype = c_int
    lib.oq_rotate_plan_build.argtypes = [vp, vp, vp, c_int, c_i64, c_i64, c_f, vp, vp]
    lib.oq_quantize_weight.restype = c_int
    lib.oq_quantize_weight.argtypes = [vp, c_int, c_i64, c_i64, vp, vp, c_int, c_i64, c_f, c_f, c_int, vp, vp, vp]
    lib.oq_rotate_quantize_mapped.restype = c_int
    lib.oq_rotate_quantize_mapped.argtypes = [vp, c_int, vp, c_i64, c_i64, vp, vp, vp, vp, c_int, c_i64, c_f, c_f, vp,
                                              vp, c_int, vp, c_int, vp, vp]
    lib.oq_debug_override.restype = c_int
    lib.oq_debug_override.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
    lib.oq_packed_linear.restype = c_int
    c_u64 = ctypes.c_uint64
    lib.oq_packed_linear.argtypes = [vp, c_int, vp, vp, c_int, vp, c_int, vp, vp, vp, c_int,
                                     c_i64, c_i64, c_i64, vp, c_int, vp, c_u64, vp]
    lib.oq_packed_linear_workspace_bytes.restype = c_u64
    lib.oq_packed_linear_workspace_bytes.argtypes = [c_i64, c_i64, c_i64, c_int, c_int, c_int]
    lib.oq_matmul_packed_weight_workspace_bytes.restype = c_u64
    lib.oq_matmul_packed_weight_workspace_bytes.argtypes = [c_i64, c_i64, c_i64, c_int, c_int]
    lib.oq_packed_linear_group.restype = c_int
    lib.oq_packed_linear_group.argtypes = [vp, c_int, vp, vp, c_int, c_int, vp, vp, vp, vp, vp, c_int,
                                           c_i64, vp, c_i64, vp, c_int, vp, c_u64, vp]
    lib.oq_packed_linear_mapped.restype = c_int
    lib.oq_packed_linear_mapped.argtypes = [vp, c_int, vp, vp, c_int, vp, c_int, vp, vp, vp, c_int,
                                            c_i64, c_i64, c_i64, vp, c_int, vp, vp, c_u64, vp]
    lib.oq_quantized_linear.restype = c_int
    lib.oq_quantized_linear.argtypes = [vp, c_int, vp, c_i64, c_i64, vp, vp, vp, vp, c_int, c_i64, c_f, c_f, vp,
                                        vp, c_int, vp, vp, vp, c_int, c_i64, vp, vp, vp, c_int, vp, vp, c_u64, vp]
    lib.oq_quantized_linear_group.restype = c_int
    lib.oq_quantized_linear_group.argtypes = [vp, c_int, vp, c_i64, c_i64, vp, vp, vp, vp, c_int, c_i64, c_f, c_f, vp,
                                              c_int, vp, vp, vp, vp, vp, c_int, vp, vp, vp, vp, c_int, vp, c_u64, vp]
    lib.oq_quantized_linear_static.restype = c_int
    lib.oq_quantized_linear_static.argtypes = [vp, c_int, vp, c_i64, c_i64, vp, vp, vp, vp, c_int, c_i64, c_f, c_f, vp,
                                               vp, c_int, vp, vp, vp, c_int, c_i64, vp, c_int, vp, vp]
    lib.oq_matmul_packed_weight.restype = c_int
    lib.oq_matmul_packed_weight.argtypes = [vp, c_int, vp, vp, c_int, vp, vp, vp, c_int,
                                            c_i64, c_i64, c_i64, vp, c_int, vp, c_u64, vp]
    lib.oq_matmul_packed_adaln_int4.restype = c_int
    lib.oq_matmul_packed_adaln_int4.argtypes = [vp, vp, vp, vp, c_i64, c_i64, c_i64, c_i64, vp, vp]
    lib.oq_quantize_adaln_weight.restype = c_int
    lib.oq_quantize_adaln_weight.argtypes = [vp, c_int, c_i64, c_i64, c_i64, vp, vp, vp]
    lib.oq_pack_lowbit.restype = c_int
    lib.oq_pack_lowbit.argtypes = [vp, c_int, c_i64, vp, vp]
    lib.oq_dequantize_packed_weight.restype = c_int
    lib.oq_dequantize_packed_weight.argtypes = [vp, c_int, vp, vp, c_i64, c_i64, vp, c_int, vp]
    lib.oq_unpack_lowbit.restype = c_int
    lib.oq_unpack_lowbit.argtypes = [vp, c_int, c_i64, vp, vp]
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        message = load().oq_last_error().decode("utf-8", "replace")
        exc = ValueError if rc == 1 else OrbitQuantHipError
        raise exc(f"{what}: {_STATUS.get(rc, rc)}: {message}")
