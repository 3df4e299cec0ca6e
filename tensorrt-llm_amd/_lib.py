"""ctypes binding of libwoq.so.  Fails loudly when the library has not been built."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# WOQ_LIB_PATH selects another build of the library (e.g. one compiled with experimental flags)
_LIB_PATH = os.environ.get("WOQ_LIB_PATH") or os.path.join(_HERE, "libwoq.so")

# enums of include/woq.h
FP16, BF16, FP8_E4M3, FP32 = 0, 1, 2, 3
W8_A16, W4_A16, W4_AFP8 = 0, 1, 2
ALGO_BIAS, ALGO_ZERO, ALGO_PRE_QUANT_SCALE, ALGO_FP8_ALPHA, ALGO_INT8_WEIGHT = 1, 2, 4, 8, 16
REGIME_AUTO, REGIME_STREAM, REGIME_GEMM = 0, 1, 2
ACT_GELU, ACT_RELU, ACT_SILU, ACT_SWIGLU, ACT_GEGLU, ACT_IDENTITY = 0, 1, 2, 3, 4, 5
ACTIVATIONS = {"gelu": ACT_GELU, "relu": ACT_RELU, "silu": ACT_SILU, "swiglu": ACT_SWIGLU, "geglu": ACT_GEGLU,
               "identity": ACT_IDENTITY}

STATUS_NAMES = {
    0: "WOQ_OK", -1: "WOQ_ERR_INVALID_ARGUMENT", -2: "WOQ_ERR_BAD_SHAPE", -3: "WOQ_ERR_UNSUPPORTED",
    -4: "WOQ_ERR_WORKSPACE", -5: "WOQ_ERR_RUNTIME", -6: "WOQ_ERR_VALUE",
}


class WoqError(RuntimeError):
    """A non-zero woq_status; `.status` holds the code (the reference raises RuntimeError from
    TORCH_CHECK / TLLM_CHECK at the same places)."""

    def __init__(self, status: int, message: str):
        super().__init__("%s: %s" % (STATUS_NAMES.get(status, str(status)), message))
        self.status = status


class MatmulArgs(ctypes.Structure):
    _fields_ = [
        ("act", ctypes.c_void_p), ("pre_quant_scale", ctypes.c_void_p), ("weight", ctypes.c_void_p),
        ("scales", ctypes.c_void_p), ("zeros", ctypes.c_void_p), ("bias", ctypes.c_void_p), ("out", ctypes.c_void_p),
        ("alpha", ctypes.c_float), ("m", ctypes.c_int32), ("n", ctypes.c_int32), ("k", ctypes.c_int32),
        ("group_size", ctypes.c_int32), ("quant_algo", ctypes.c_int32), ("act_dtype", ctypes.c_int32),
        ("out_dtype", ctypes.c_int32), ("regime", ctypes.c_int32), ("workspace", ctypes.c_void_p),
        ("workspace_bytes", ctypes.c_size_t),
    ]


class GroupedMatmulArgs(ctypes.Structure):
    _fields_ = [("base", MatmulArgs), ("total_rows_before_expert", ctypes.c_void_p), ("num_experts", ctypes.c_int32),
                ("activation", ctypes.c_int32), ("residual", ctypes.c_void_p)]


def lib_path() -> str:
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        raise ImportError(
            "libwoq.so is not built (%s). Build it with `python tensorrt-llm_amd/build.py`; "
            "there is no fallback implementation." % _LIB_PATH)
    lib = ctypes.CDLL(_LIB_PATH)
    vp, i32, i64, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_size_t
    sig = {
        "woq_matmul": (ctypes.c_int, [ctypes.POINTER(MatmulArgs), vp]),
        "woq_matmul_check": (ctypes.c_int, [ctypes.POINTER(MatmulArgs)]),
        "woq_matmul_static": (ctypes.c_int, [ctypes.POINTER(MatmulArgs), vp]),
        "woq_static_scratch_bytes": (sz, []),
        "woq_static_init": (ctypes.c_int, []),
        "woq_grouped_matmul": (ctypes.c_int, [ctypes.POINTER(GroupedMatmulArgs), vp]),
        "woq_grouped_matmul_check": (ctypes.c_int, [ctypes.POINTER(GroupedMatmulArgs)]),
        "woq_workspace_bytes": (sz, [i32, i32, i32, i32, i32]),
        "woq_select_regime": (ctypes.c_int, [i32, i32, i32, i32]),
        "woq_preprocessed_bytes": (sz, [i64, i64, i32]),
        "woq_preprocess_weights": (ctypes.c_int, [vp, vp, i64, i64, i64, i32]),
        "woq_unpreprocess_weights": (ctypes.c_int, [vp, vp, i64, i64, i64, i32]),
        "woq_import_reference_weights": (ctypes.c_int, [vp, vp, i64, i64, i64, i32, i32]),
        "woq_reference_layout_step": (ctypes.c_int, [vp, vp, i64, i64, i64, i32, i32]),
        "woq_symmetric_quantize": (ctypes.c_int, [vp, vp, vp, vp, i64, i64, i64, i32, i32, i32]),
        "woq_pack_int4": (ctypes.c_int, [vp, vp, sz]),
        "woq_unpack_int4": (ctypes.c_int, [vp, vp, sz]),
        "woq_apply_per_channel_scale": (ctypes.c_int, [vp, vp, vp, i32, i32, i32, i32, vp]),
        "woq_rmsnorm_prequant": (ctypes.c_int, [vp, vp, vp, vp, vp, ctypes.c_float, i32, i32, i32, i32, vp]),
        "woq_dequantize": (ctypes.c_int, [vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]),
        "woq_profile_tactics": (ctypes.c_int, [ctypes.POINTER(MatmulArgs), i32, i32, vp]),
        "woq_tactic_count": (ctypes.c_int, []),
        "woq_clear_tactics": (None, []),
        "woq_describe_tactic": (ctypes.c_int, [ctypes.POINTER(MatmulArgs), ctypes.c_char_p, sz]),
        "woq_export_tactics": (sz, [ctypes.c_char_p, sz]),
        "woq_import_tactics": (ctypes.c_int, [ctypes.c_char_p]),
        "woq_reload_env": (None, []),
        "woq_last_error": (ctypes.c_char_p, []),
        "woq_last_launch": (ctypes.c_char_p, []),
        "woq_abi_version": (ctypes.c_int, []),
        "woq_layout_version": (ctypes.c_int, []),
    }
    # measurement probes (csrc/woq_probes.h): in the library, outside the drop-in boundary
    probes = {
        "woq_probe_read": (ctypes.c_int, [vp, sz, i32, i32, vp, vp]),
        "woq_probe_empty": (ctypes.c_int, [vp, vp]),
        "woq_probe_mfma": (ctypes.c_double, [i32, i32, i32, i32, vp, vp]),
    }
    for table in (sig, probes):
        for name, (res, args) in table.items():
            fn = getattr(lib, name)  # AttributeError here = header and library disagree
            fn.restype = res
            fn.argtypes = args
    return lib, tuple(sig), tuple(probes)


lib, EXPORTED, PROBES = _load()


def check(status: int) -> None:
    if status != 0:
        raise WoqError(status, (lib.woq_last_error() or b"").decode())
