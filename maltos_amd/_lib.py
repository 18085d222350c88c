"""ctypes binding of libmaltos_hip.so (the C ABI declared in include/maltos_hip.h).

There is no CPU fallback anywhere in this package: if the library is missing, `lib()` raises and
so does every op.  torch is imported first so that the library's libamdhip64.so.7 dependency
resolves to the HIP runtime torch already loaded (one runtime per process, shared streams).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

import torch  # noqa: F401  (must precede CDLL, see module docstring)

LIB_PATH = Path(__file__).resolve().parent / "libmaltos_hip.so"

MLTS_OK = 0
MLTS_ERR_INVALID = 1
MLTS_ERR_UNSUPPORTED = 2
MLTS_ERR_LAUNCH = 3

MLTS_F32 = 0
MLTS_BF16 = 1

MASK_NONE = 0
MASK_CAUSAL = 1
MASK_DOC = 2

SQNORM_WS_BYTES = 16384

_i64x3 = C.c_int64 * 3


class AttnShape(C.Structure):
    """Mirror of `struct mlts_attn_shape`."""

    _fields_ = [
        ("B", C.c_int32),
        ("Hq", C.c_int32),
        ("Hkv", C.c_int32),
        ("Sq", C.c_int32),
        ("Sk", C.c_int32),
        ("D", C.c_int32),
        ("dtype", C.c_int32),
        ("mask_mode", C.c_int32),
        ("scale", C.c_float),
        ("q_stride", _i64x3),
        ("k_stride", _i64x3),
        ("v_stride", _i64x3),
        ("o_stride", _i64x3),
        ("q_pos", C.c_void_p),
        ("k_pos", C.c_void_p),
        ("q_seq", C.c_void_p),
        ("k_seq", C.c_void_p),
        ("doc_plan", C.c_void_p),
    ]


_P = C.c_void_p
_I64P = C.POINTER(C.c_int64)
_SHAPE_P = C.POINTER(AttnShape)

# name -> (restype, argtypes); one entry per function declared in include/maltos_hip.h
SIGNATURES: dict[str, tuple[object, list[object]]] = {
    "mlts_abi_version": (C.c_int, []),
    "mlts_last_error": (C.c_char_p, []),
    "mlts_kernel_timing_enable": (None, [C.c_int]),
    "mlts_kernel_timing_read": (C.c_int, [C.c_char_p, C.POINTER(C.c_double), C.POINTER(C.c_int64)]),
    "mlts_attn_supports": (C.c_char_p, [_SHAPE_P]),
    "mlts_attn_doc_plan_bytes": (C.c_int64, [_SHAPE_P]),
    "mlts_attn_doc_plan": (C.c_int, [_SHAPE_P, _P, C.c_int64, _P]),
    "mlts_attn_fwd_workspace_bytes": (C.c_int64, [_SHAPE_P]),
    "mlts_attn_bwd_workspace_bytes": (C.c_int64, [_SHAPE_P, C.c_int]),
    "mlts_attn_fwd": (C.c_int, [_SHAPE_P, _P, _P, _P, _P, _P, _P, C.c_int64, _P]),
    "mlts_attn_bwd": (
        C.c_int,
        [_SHAPE_P, _P, _I64P, _P, _P, _P, _P, _P, _P, _I64P, _P, _I64P, _P, _I64P, C.c_int, _P, C.c_int64, _P],
    ),
    "mlts_attn_bwd_noalloc": (
        C.c_int,
        [_SHAPE_P, _P, _I64P, _P, _P, _P, _P, _P, _P, _I64P, _P, _I64P, _P, _I64P, C.c_int, _P],
    ),
    "mlts_attn_merge": (
        C.c_int,
        [_P, _P, _P, _I64P, C.c_int32, _P, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, _P],
    ),
    "mlts_rmsnorm_fwd": (C.c_int, [_P, _P, _P, _P, C.c_int64, C.c_int32, C.c_float, C.c_int32, _P]),
    "mlts_rmsnorm_bwd_workspace_bytes": (C.c_int64, [C.c_int64, C.c_int32]),
    "mlts_rmsnorm_bwd": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, C.c_int64, C.c_int64, C.c_int32, C.c_int32, _P]),
    "mlts_add_rmsnorm_fwd": (C.c_int, [_P, _P, _P, _P, _P, _P, C.c_int64, C.c_int32, C.c_float, C.c_int32, _P]),
    "mlts_add_rmsnorm_bwd": (C.c_int, [_P, _P, _P, _P, _P, _P, _P, _P, C.c_int64, C.c_int64, C.c_int32, C.c_int32, _P]),
    "mlts_rope": (
        C.c_int,
        [_P, _I64P, _P, _I64P, _P, _P, C.c_int32, _P, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32,
         C.c_int32, C.c_int32, _P],
    ),
    "mlts_rope_pair": (
        C.c_int,
        [_P, _I64P, _P, _I64P, C.c_int32, _P, _I64P, _P, _I64P, C.c_int32, _P, _P, C.c_int32, _P, C.c_int32, C.c_int32,
         C.c_int32, C.c_int32, C.c_int32, C.c_int32, _P],
    ),
    "mlts_swiglu_fwd": (C.c_int, [_P, _P, _P, C.c_int64, C.c_int32, _P]),
    "mlts_swiglu_bwd": (C.c_int, [_P, _P, _P, _P, _P, C.c_int64, C.c_int32, _P]),
    "mlts_swiglu_fwd_rows": (C.c_int, [_P, _P, C.c_int64, _P, C.c_int64, C.c_int64, C.c_int64, C.c_int32, _P]),
    "mlts_swiglu_bwd_rows": (C.c_int, [_P, C.c_int64, _P, _P, C.c_int64, _P, _P, C.c_int64, C.c_int64, C.c_int64, C.c_int32, _P]),
    "mlts_ce_workspace_bytes": (C.c_int64, [C.c_int64]),
    "mlts_ce_fwd_bwd": (C.c_int, [_P, _P, _P, _P, _P, _P, C.c_int64, C.c_int64, C.c_int32, C.c_int64, C.c_int32, _P]),
    "mlts_scale_by_device_scalar": (C.c_int, [_P, _P, C.c_int64, C.c_int32, _P]),
    "mlts_grad_to_f32": (C.c_int, [_P, _P, C.c_int32, C.c_int64, C.c_int, _P, _P, _P]),
    "mlts_grad_sum_slices": (C.c_int, [_P, _P, C.c_int32, C.c_int32, C.c_int64, C.c_int, _P]),
    "mlts_sq_norm": (C.c_int, [_P, C.c_int64, _P, _P, _P]),
    "mlts_scale": (C.c_int, [_P, C.c_float, C.c_int64, _P]),
    "mlts_adamw_step": (
        C.c_int,
        [_P, _P, _P, _P, _P, C.c_int64, C.c_float, C.c_float, C.c_float, C.c_float, C.c_float, C.c_int64, C.c_float,
         _P, C.c_float, _P],
    ),
}

_LIB: C.CDLL | None = None


class MaltosHipError(RuntimeError):
    """The native library is missing, or a kernel entry point reported a launch failure."""


def lib() -> C.CDLL:
    global _LIB
    if _LIB is not None:
        return _LIB
    if not LIB_PATH.exists():
        raise MaltosHipError(
            f"{LIB_PATH} is missing: build it with `python -m maltos_amd.build`. "
            "maltos_amd has no CPU or eager fallback."
        )
    handle = C.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(handle, name, None)
        if fn is None:
            raise MaltosHipError(f"{LIB_PATH} does not export {name}; rebuild it")
        fn.restype = restype
        fn.argtypes = argtypes
    _LIB = handle
    return handle


def last_error() -> str:
    msg = lib().mlts_last_error()
    return msg.decode("utf-8", "replace") if msg else ""


def check(status: int) -> None:
    """Translate a status code into the exception type the reference would raise."""
    if status == MLTS_OK:
        return
    msg = last_error()
    if status == MLTS_ERR_INVALID:
        raise ValueError(msg)
    if status == MLTS_ERR_UNSUPPORTED:
        raise RuntimeError(msg)
    raise MaltosHipError(msg or f"libmaltos_hip status {status}")


def kernel_timing(enable: bool) -> None:
    lib().mlts_kernel_timing_enable(int(enable))


def kernel_time_ms(name: str) -> tuple[float, int]:
    """(summed kernel milliseconds, launches) recorded for `name` since timing was enabled."""
    total, count = C.c_double(0.0), C.c_int64(0)
    check(lib().mlts_kernel_timing_read(name.encode(), C.byref(total), C.byref(count)))
    return total.value, count.value


def strides3(values) -> C.Array:
    return _i64x3(*[int(v) for v in values])
