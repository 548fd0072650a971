"""ctypes binding of libdtas_gfx950.so (the C ABI declared in include/dtas_abi.h).

The library is the product: there is no Python or CPU fallback.  If the shared object is
missing, ``lib()`` raises with the build command instead of computing anything elsewhere.
"""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# DTAS_LIBRARY: another build of the same library (same ABI), e.g. one made with other compile-time constants to be
# measured beside the product's; unset, the library built in-tree next to this file
LIB_PATH = os.environ.get("DTAS_LIBRARY") or os.path.join(_HERE, "libdtas_gfx950.so")

ABI_VERSION = 1

# enum dtas_op
(OP_ADD_F16, OP_ADD_F32, OP_ADD_I8, OP_COPY_F16, OP_COPY_F32, OP_COPY_I8, OP_CAST_F16_F32, OP_CAST_F32_F16,
 OP_LAYER_NORM_F32_F16, OP_RMS_NORM_F16, OP_SOFTMAX_F32_F16, OP_SOFTMAX_F16, OP_GEMV_F16, OP_GEMM_F16,
 OP_COUNT) = range(15)

# enum dtas_variant
ELT_VECTOR, ELT_SCALAR = 0, 1
RED_WAVE_ROW, RED_BLOCK_ROW, RED_STREAM_ROW = 0, 1, 2
GEMV_SPLITK, GEMV_RF16 = 0, 1
GEMM_MFMA, GEMM_SKINNY, GEMM_ROWS, GEMM_STREAM, GEMM_MFMA_ACC16 = 0, 1, 2, 3, 4
# enum dtas_epilogue
EPI_BIAS, EPI_BIAS_ADD2, EPI_BIAS_ADD2_CAST_F32, EPI_BIAS_GELU = 0, 1, 2, 3


class DtasConfig(ctypes.Structure):
    """struct dtas_config: one row of a call table."""

    _fields_ = [
        ("variant", ctypes.c_int32),
        ("block", ctypes.c_int32),
        ("vec", ctypes.c_int32),
        ("unroll", ctypes.c_int32),
        ("tile", ctypes.c_int32 * 3),
        ("split_k", ctypes.c_int32),
        ("grid_cap", ctypes.c_int64),
    ]

    def to_dict(self) -> dict:
        return {"variant": self.variant, "block": self.block, "vec": self.vec, "unroll": self.unroll,
                "tile": list(self.tile), "split_k": self.split_k, "grid_cap": self.grid_cap}

    @classmethod
    def from_dict(cls, d: dict) -> "DtasConfig":
        c = cls()
        c.variant, c.block, c.vec, c.unroll = d["variant"], d["block"], d["vec"], d["unroll"]
        t = list(d.get("tile", [0, 0, 0])) + [0, 0, 0]
        c.tile[0], c.tile[1], c.tile[2] = t[0], t[1], t[2]
        c.split_k = d.get("split_k", 1)
        c.grid_cap = d.get("grid_cap", 0)
        return c


class DtasLaunchInfo(ctypes.Structure):
    """struct dtas_launch_info: what the dispatcher decided for one call."""

    _fields_ = [
        ("launch_args", ctypes.c_int64 * 7),
        ("bucket_lo", ctypes.c_int64),
        ("bucket_hi", ctypes.c_int64),
        ("index", ctypes.c_int32),
        ("table_row", ctypes.c_int32),
        ("config", DtasConfig),
        ("name", ctypes.c_char * 96),
    ]


_vp, _i64, _f32, _ci = ctypes.c_void_p, ctypes.c_int64, ctypes.c_float, ctypes.c_int
_cfg = ctypes.POINTER(DtasConfig)

# name -> argtypes; every entry point returns int (0 ok / -1 error)
SIGNATURES = {
    "dtas_abi_version": [],
    "dtas_init": [],
    "dtas_select_bucket": [_ci, _i64, _i64, _i64, ctypes.POINTER(DtasLaunchInfo)],
    "dtas_describe_launch": [_ci, _i64, _i64, _i64, _cfg, ctypes.POINTER(DtasLaunchInfo)],
    "dtas_add_f16": [_vp, _vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_add_f32": [_vp, _vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_add_i8": [_vp, _vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_copy_f16": [_vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_copy_f32": [_vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_copy_i8": [_vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_cast_f16_f32": [_vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_cast_f32_f16": [_vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_layer_norm_f32_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _f32, _cfg, _vp],
    "dtas_rms_norm_f16": [_vp, _vp, _vp, _i64, _i64, _f32, _cfg, _vp],
    "dtas_softmax_f32_f16": [_vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_softmax_f16": [_vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_gemv_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_gemv_f16_fused": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, ctypes.c_int32, _cfg, _vp],
    "dtas_gemm_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _cfg, _vp],
    "dtas_gemm_f16_static": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _cfg, _vp],
    "dtas_gemm_f16_fused": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_int32, _cfg, _vp],
    "dtas_attn_scores_f16_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, ctypes.c_float, _cfg, _vp],
    "dtas_attn_pv_f16": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _cfg, _vp],
    "dtas_gemv_f32": [_vp, _vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_decode_q8_f16": [_vp, _vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_gemv_q8_f16": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, ctypes.c_int32, _cfg, _vp],
    "dtas_attn_mask_f16": [_vp, _i64, _i64, _vp],
    "dtas_swap_axes_f16": [_vp, _vp, _i64, _i64, _i64, _vp],
    "dtas_split3_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _vp],
    "dtas_softmax_temperature_f32": [_vp, _vp, _vp, _i64, _i64, _vp],
    "dtas_divide_f32": [_vp, _vp, _vp, _i64, _vp],
    "dtas_layer_norm_f32": [_vp, _vp, _vp, _vp, _i64, _i64, ctypes.c_float, _vp],
    "dtas_softmax_f32": [_vp, _vp, _i64, _i64, _vp],
    "dtas_rotary_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _cfg, _vp],
    "dtas_take_f16": [_vp, _vp, _vp, _i64, _i64, _i64, _cfg, _vp],
    "dtas_take_q8_f16": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _cfg, _vp],
    "dtas_gemv_q8_f32": [_vp, _vp, _vp, _vp, _i64, _i64, _cfg, _vp],
    "dtas_gemm_q8_f16_fused": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, ctypes.c_int32, _cfg, _vp],
}

_lib = None


class DtasError(RuntimeError):
    """An entry point returned -1; the message is dtas_last_error()."""


def lib() -> ctypes.CDLL:
    """The loaded library.  Raises if it has not been built: nothing else can stand in for it."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.join(_HERE, 'csrc')}` "
                "(hipcc --offload-arch=gfx950); dtas_amd has no fallback path")
        handle = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        handle.dtas_last_error.argtypes = []
        handle.dtas_last_error.restype = ctypes.c_char_p
        if handle.dtas_abi_version() != ABI_VERSION:
            raise ImportError(f"{LIB_PATH}: ABI version {handle.dtas_abi_version()} != {ABI_VERSION}")
        _lib = handle
    return _lib


def last_error() -> str:
    return lib().dtas_last_error().decode("utf-8", "replace")


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise DtasError(f"{what}: {last_error()}")


def select_bucket(op: int, n: int, d0: int = 0, d1: int = 0) -> DtasLaunchInfo:
    info = DtasLaunchInfo()
    check(lib().dtas_select_bucket(op, n, d0, d1, ctypes.byref(info)), "dtas_select_bucket")
    return info


def describe_launch(op: int, n: int, d0: int, d1: int, cfg: DtasConfig) -> DtasLaunchInfo:
    info = DtasLaunchInfo()
    check(lib().dtas_describe_launch(op, n, d0, d1, ctypes.byref(cfg), ctypes.byref(info)), "dtas_describe_launch")
    return info
