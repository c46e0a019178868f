"""ctypes binding of the C-ABI HIP library (include/calibquant_hip.h).

The library is built in-tree by `python -m calibquant_amd.build`.  There is no
CPU fallback: if the library is missing, loading raises."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# CALIBQUANT_HIP_LIBRARY: another build of the same C ABI (the profiling build with phase stops,
# `python -m calibquant_amd.build --phase-stops`); default: the library built in-tree
LIB_PATH = os.environ.get("CALIBQUANT_HIP_LIBRARY") or os.path.join(_HERE, "lib", "libcalibquant_hip.so")

CQ_BF16, CQ_FP16, CQ_FP32, CQ_I64, CQ_I32, CQ_U8 = range(6)

SYMBOLS = (
    "cq_version", "cq_strerror", "cq_last_hip_error",
    "cq_quantize_pack_workspace", "cq_quantize_pack", "cq_rope_quantize_pack", "cq_rope_rows", "cq_rope_rows_grouped", "cq_quant", "cq_quant_tensor", "cq_encode",
    "cq_lut_vecmat_qk", "cq_lut_vecmat_pv",
    "cq_decode_attn_workspace", "cq_decode_attn", "cq_decode_attn_static", "cq_decode_attn_static_limit",
    "cq_decode_attn_plan", "cq_decode_attn_wait_polls", "cq_decode_attn_gave_up", "cq_quantize_pack_wait_polls", "cq_decode_attn_single_launch", "cq_rope_append", "cq_quantize_pack_token",
)


class DecodePlan(C.Structure):
    """Mirror of `cq_decode_plan`."""
    _fields_ = [("threads", C.c_int), ("heads_per_unit", C.c_int), ("chunks", C.c_int), ("chunk_tokens", C.c_int),
                ("launches", C.c_int), ("lds_bytes", C.c_int), ("register_logits", C.c_int)]


class DecodeArgs(C.Structure):
    """Mirror of `cq_decode_args`."""
    _fields_ = [
        ("q", C.c_void_p),
        ("codes_k", C.c_void_p), ("codes_v", C.c_void_p),
        ("k_scale", C.c_void_p), ("k_zero", C.c_void_p),
        ("v_scale", C.c_void_p), ("v_zero", C.c_void_p),
        ("k_res", C.c_void_p), ("v_res", C.c_void_p),
        ("res_stride_b", C.c_int64), ("res_stride_h", C.c_int64), ("res_stride_r", C.c_int64),
        ("mask", C.c_void_p), ("mask_stride_b", C.c_int64),
        ("out", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("dtype", C.c_int),
        ("B", C.c_int), ("Hq", C.c_int), ("Hkv", C.c_int), ("D", C.c_int),
        ("T", C.c_int), ("R", C.c_int), ("sprompt_len", C.c_int), ("bits", C.c_int),
        ("calibrate", C.c_int), ("calib_off_max", C.c_float), ("calib_off_min", C.c_float),
        ("force_splits", C.c_int),
        ("r_dev", C.c_void_p),
        ("v_mode", C.c_int),
    ]


class CalibQuantError(RuntimeError):
    pass


_lib = None


def load() -> C.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise CalibQuantError(
            f"{LIB_PATH} is missing: build it with `python -m calibquant_amd.build` "
            "(there is no CPU fallback for these operators)")
    lib = C.CDLL(LIB_PATH)
    i, i64, vp, sz, f = C.c_int, C.c_int64, C.c_void_p, C.c_size_t, C.c_float
    lib.cq_version.restype = i
    lib.cq_strerror.restype = C.c_char_p
    lib.cq_strerror.argtypes = [i]
    lib.cq_last_hip_error.restype = i
    lib.cq_quantize_pack_workspace.restype = sz
    lib.cq_quantize_pack_workspace.argtypes = [i, i, i, i]
    qargs = [vp, i, i, i, i, i, i64, i64, i64, i, f, vp, vp, vp, vp, sz, vp]
    lib.cq_quantize_pack.restype = i
    lib.cq_quantize_pack.argtypes = qargs
    lib.cq_quant.restype = i
    lib.cq_quant.argtypes = qargs
    rope_common = [vp, i, i, i, i, i, i64, i64, i64, vp, vp, i64, vp, i64, i64, i64, vp, i64, i64, i64]
    lib.cq_rope_quantize_pack.restype = i
    lib.cq_rope_quantize_pack.argtypes = rope_common + [i, f, vp, vp, vp, vp, sz, vp]
    lib.cq_rope_rows.restype = i
    lib.cq_rope_rows.argtypes = rope_common + [vp]
    lib.cq_rope_rows_grouped.restype = i
    lib.cq_rope_rows_grouped.argtypes = [vp, i, i, i, i, i, i, i64, i64, i64, i64, vp, vp, i64, vp, i64, i64, i64,
                                         vp, i64, i64, i64, i64, vp]
    lib.cq_quant_tensor.restype = i
    lib.cq_quant_tensor.argtypes = qargs
    lib.cq_encode.restype = i
    lib.cq_encode.argtypes = [vp, i, i64, i, i, vp, vp]
    vm = [vp, i, i, vp, i, vp, i64, i, i, i, vp, vp]
    lib.cq_lut_vecmat_qk.restype = i
    lib.cq_lut_vecmat_qk.argtypes = vm
    lib.cq_lut_vecmat_pv.restype = i
    lib.cq_lut_vecmat_pv.argtypes = vm
    lib.cq_decode_attn_workspace.restype = sz
    lib.cq_decode_attn_workspace.argtypes = [C.POINTER(DecodeArgs)]
    lib.cq_decode_attn_plan.restype = C.c_int
    lib.cq_decode_attn_plan.argtypes = [C.POINTER(DecodeArgs), C.POINTER(DecodePlan)]
    lib.cq_decode_attn.restype = i
    lib.cq_decode_attn.argtypes = [C.POINTER(DecodeArgs), vp]
    lib.cq_decode_attn_wait_polls.restype = i
    lib.cq_decode_attn_wait_polls.argtypes = [i]
    lib.cq_quantize_pack_wait_polls.restype = i
    lib.cq_quantize_pack_wait_polls.argtypes = [i]
    lib.cq_decode_attn_gave_up.restype = i
    lib.cq_decode_attn_gave_up.argtypes = []
    lib.cq_decode_attn_single_launch.restype = i
    lib.cq_decode_attn_single_launch.argtypes = [i]
    lib.cq_decode_attn_static.restype = i
    lib.cq_decode_attn_static.argtypes = [C.POINTER(DecodeArgs), vp]
    lib.cq_decode_attn_static_limit.restype = sz
    lib.cq_decode_attn_static_limit.argtypes = []
    lib.cq_quantize_pack_token.restype = i
    lib.cq_quantize_pack_token.argtypes = [vp, i, i, i, i, i, i64, i64, i64, i, i, vp, vp, vp, vp]
    lib.cq_rope_append.restype = i
    lib.cq_rope_append.argtypes = [vp, i, i, i, i, i, vp, vp, i64, vp, i64, vp, vp, vp, i64, i64, i64, i, vp, vp]
    _lib = lib
    return lib


SHIM_PATH = os.path.join(_HERE, "lib", "_cq_torch_step.so")
_shim = None


def load_step_shim():
    """The host shim `_cq_torch_step` (C++ over torch's headers; `LayerStep` runs the steady-state decode
    step of one attention layer in one call).  Built by `python -m calibquant_amd.build`; raises if missing."""
    global _shim
    if _shim is None:
        if not os.path.exists(SHIM_PATH):
            raise CalibQuantError(f"{SHIM_PATH} is missing: build it with `python -m calibquant_amd.build`")
        import importlib.util

        import torch  # noqa: F401  (the shim links torch's libraries; they must be loaded first)
        load()
        spec = importlib.util.spec_from_file_location("_cq_torch_step", SHIM_PATH)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        if mod.library_version() != load().cq_version():
            raise CalibQuantError("the host shim and the HIP library were built from different sources")
        _shim = mod
    return _shim


def check(status: int, what: str) -> None:
    if status != 0:
        lib = load()
        msg = lib.cq_strerror(status).decode()
        extra = f" (hipError {lib.cq_last_hip_error()})" if status == -6 else ""
        raise CalibQuantError(f"{what}: {msg}{extra}")
