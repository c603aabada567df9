"""ctypes binding of libmoe_i8.so (the C-ABI declared in include/moe_i8.h).

The library is loaded from the package directory only.  There is no fallback: if it has not been
built, or exports fewer symbols than the header declares, importing callers get an error.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from pathlib import Path

PKG_DIR = Path(__file__).resolve().parent
LIB_PATH = PKG_DIR / "libmoe_i8.so"
PROBE_LIB_PATH = PKG_DIR / "libmoe_i8_probe.so"  # benchmark aid, not part of the product ABI

OK = 0
EINVAL, EWORKSPACE, ELAUNCH, EUNSUPPORTED = -1, -2, -3, -4
DTYPE_BF16 = 0
GEMM_AUTO, GEMM_STREAM, GEMM_TILE, GEMM_NARROW, GEMM_TILE_WIDE, GEMM_TILE_DEEP, GEMM_TILE_RING = 0, 1, 2, 3, 4, 5, 6
SCORE_SOFTMAX, SCORE_SIGMOID, SCORE_TOPK_SOFTMAX = 0, 1, 2
MAX_EXPERTS = 1024

_P = c_void_p
# name -> (restype, argtypes); mirrors include/moe_i8.h one to one
SIGNATURES = {
    "moe_i8_version": (c_int, []),
    "moe_i8_last_error": (c_char_p, []),
    "moe_i8_sorted_capacity": (c_int64, [c_int64, c_int, c_int]),
    "moe_i8_align_workspace_bytes": (c_int64, [c_int64, c_int, c_int]),
    "moe_i8_align_block_size": (c_int, [_P, c_int64, c_int, c_int, _P, c_int64, _P, c_int64, _P, _P, c_int64, _P]),
    "moe_i8_quant_rows": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, c_int, c_int64, _P, _P, _P]),
    "moe_i8_gemm_down_bf16": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int64, _P, _P],
    ),
    "moe_i8_scaled_int8_quant": (c_int, [_P, c_int, c_int64, c_int64, c_int64, _P, _P, _P]),
    "moe_i8_dense_workspace_bytes": (c_int64, [c_int64, c_int, c_int]),
    "moe_i8_w8a8_linear": (c_int, [_P, _P, _P, _P, c_int64, c_int, c_int, _P, c_int64, c_int, _P]),
    "moe_i8_w8a8_mlp": (c_int, [_P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, _P, c_int64, c_int, _P]),
    "moe_i8_route_topk": (
        c_int,
        [_P, c_int64, c_int, c_int, c_int, _P, c_int, c_int, c_int, c_int, c_float, _P, _P, _P, c_int, c_int64,
         c_int64, _P],
    ),
    "moe_i8_quant_weights": (c_int, [_P, c_int, c_int64, c_int64, c_int64, c_int64, c_int64, _P, _P, _P]),
    "moe_i8_gemm_gate_up_silu": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, c_int64, _P, c_int, _P],
    ),
    "moe_i8_gemm_down": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int64, _P, c_int, _P],
    ),
    "moe_i8_gemm_acc_i32": (
        c_int,
        [_P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, c_int64, _P, c_int, _P],
    ),
    "moe_i8_sum": (c_int, [_P, _P, c_int64, c_int, c_int, _P]),
    "moe_i8_workspace_bytes": (c_int64, [c_int64, c_int, c_int, c_int, c_int, c_int]),
    "moe_i8_fused_experts": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, _P, c_int64, c_int, _P],
    ),
    "moe_i8_layer_plan": (c_int, [c_int64, c_int, c_int, c_int, c_int, c_int, c_int, _P, _P, _P]),
    "moe_i8_fused_experts_static": (
        c_int,
        [_P, _P, _P, _P, _P, _P, _P, _P, c_int64, c_int, c_int, c_int, c_int, c_int, c_int, _P],
    ),
}
STATIC_SCRATCH_BYTES = 32 << 20

_lib = None


class MoeI8Error(RuntimeError):
    """A C-ABI call returned a non-zero code."""

    def __init__(self, code: int, message: str):
        super().__init__(f"libmoe_i8 error {code}: {message}")
        self.code = code


def load() -> ctypes.CDLL:
    """Load the library once and bind every declared symbol; raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "(there is no CPU or PyTorch fallback for this path)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def check(code: int) -> None:
    if code != OK:
        raise MoeI8Error(code, load().moe_i8_last_error().decode("utf-8", "replace"))
