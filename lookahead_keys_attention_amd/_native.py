"""ctypes binding of libcastle_hip.so (C ABI in include/castle_hip.h).

The library is looked up next to this file only.  Nothing here falls back to another
implementation: if the library is missing or a call fails, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libcastle_hip.so")

ABI_VERSION = 5
DTYPE_CODES = {torch.float32: 0, torch.bfloat16: 1, torch.float16: 2}
SUPPORTED_HEAD_DIMS = (16, 32, 64, 128)
FLAG_BF16_OPERANDS = 1   # keep bf16 MFMA operands for bf16 tensors (default: fp16 operands)
FLAG_ROTARY = 2          # rotary position embedding of qc, kc, qu, ku, vu inside the kernels
FLAG_RECOMPUTE_SCORES = 4   # backward without the dS / dSu tile hand-over (less workspace, slower)
FLAG_RECOMPUTE_STATE = 8    # backward re-runs the forward scan: the forward state buffer need not be kept
FLAG_U_HALF = 16            # bf16 caches: the lookahead-key buffer holds fp16 bits of U / 64 (see castle_hip.h)
U_HALF_UNSCALE = 64.0

EXPORTED_SYMBOLS = (
    "castle_abi_version",
    "castle_error_string",
    "castle_fwd_workspace_bytes",
    "castle_fwd_state_bytes",
    "castle_fwd",
    "castle_bwd_workspace_bytes",
    "castle_bwd",
    "castle_decode_workspace_bytes",
    "castle_decode_step",
    "castle_decode_step_device_count",
    "castle_decode_step_static",
    "castle_decode_flush",
    "castle_rope",
    "castle_small_linear",
    "castle_small_linear_fused",
    "castle_profile_enable",
    "castle_profile_read",
)


class View4(ctypes.Structure):
    """struct castle_view4"""

    _fields_ = [
        ("ptr", ctypes.c_void_p),
        ("stride_b", ctypes.c_int64),
        ("stride_h", ctypes.c_int64),
        ("stride_l", ctypes.c_int64),
    ]


class Deferred(ctypes.Structure):
    """struct castle_deferred"""

    _fields_ = [
        ("vu_ring", View4),
        ("gates", View4),
        ("base", ctypes.c_int32),
        ("base_device", ctypes.c_void_p),
    ]


DECODE_DEFER = 4   # U is written on every 4th step when a castle_deferred is handed over
_VP = ctypes.POINTER(View4)
_DP = ctypes.POINTER(Deferred)
_lib = None
_lock = threading.Lock()


def _declare(lib):
    i, i64, f, vp = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p
    lib.castle_abi_version.restype = i
    lib.castle_abi_version.argtypes = []
    lib.castle_error_string.restype = ctypes.c_char_p
    lib.castle_error_string.argtypes = [i]
    lib.castle_fwd_workspace_bytes.restype = i64
    lib.castle_fwd_workspace_bytes.argtypes = [i, i, i, i, i]
    lib.castle_fwd_state_bytes.restype = i64
    lib.castle_fwd_state_bytes.argtypes = [i, i, i, i, i]
    lib.castle_bwd_workspace_bytes.restype = i64
    lib.castle_bwd_workspace_bytes.argtypes = [i, i, i, i, i, i]
    lib.castle_decode_workspace_bytes.restype = i64
    lib.castle_decode_workspace_bytes.argtypes = [i, i, i, i]
    lib.castle_fwd.restype = i
    lib.castle_fwd.argtypes = [_VP] * 6 + [i, i, i, i, i, f, i, _VP, _VP, vp, i64, vp, i64, vp]
    lib.castle_bwd.restype = i
    lib.castle_bwd.argtypes = [_VP] * 8 + [i, i, i, i, i, f, i] + [_VP] * 6 + [vp, i64, vp, i64, vp, i64, vp]
    lib.castle_profile_enable.restype = i
    lib.castle_profile_enable.argtypes = [i]
    lib.castle_profile_read.restype = i
    lib.castle_profile_read.argtypes = [ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_float), i]
    lib.castle_decode_step.restype = i
    lib.castle_decode_step.argtypes = [_VP] * 4 + [i, i] + [_VP] * 6 + [i, i, i, i, f, i, _VP, _DP, vp, i64, vp]
    lib.castle_decode_step_static.restype = i
    lib.castle_decode_step_static.argtypes = [_VP] * 4 + [i, vp, i] + [_VP] * 6 + [i, i, i, i, f, i, _VP, _DP, vp]
    lib.castle_decode_flush.restype = i
    lib.castle_decode_flush.argtypes = [_VP, _VP, i, _DP, i, i, i, i, f, i, vp]
    lib.castle_decode_step_device_count.restype = i
    lib.castle_decode_step_device_count.argtypes = [_VP] * 4 + [vp, i] + [_VP] * 6 + [i, i, i, i, f, i, _VP, _DP, vp, i64, vp]
    lib.castle_small_linear.restype = i
    lib.castle_small_linear.argtypes = [vp, vp, vp, i, i, i, i64, i64, i64, i, vp]
    lib.castle_small_linear_fused.restype = i
    lib.castle_small_linear_fused.argtypes = [vp, vp, vp, i, i, i, i64, i64, i64, i, vp, ctypes.c_float, i, vp, i64, vp]
    lib.castle_rope.restype = i
    lib.castle_rope.argtypes = [_VP, _VP, i, i, i, i, i, i, vp]


def lib():
    """The loaded library (loads it on first use; raises if it has not been built)."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                if not os.path.exists(LIB_PATH):
                    raise RuntimeError(
                        f"{LIB_PATH} not found: build the HIP kernels first "
                        "(python -m lookahead_keys_attention_amd.build)"
                    )
                handle = ctypes.CDLL(LIB_PATH)
                _declare(handle)
                got = handle.castle_abi_version()
                if got != ABI_VERSION:
                    raise RuntimeError(f"libcastle_hip.so has ABI {got}, this package needs {ABI_VERSION}")
                _lib = handle
    return _lib


def is_built() -> bool:
    return os.path.exists(LIB_PATH)


def check(code: int, what: str):
    if code < 0:
        msg = lib().castle_error_string(int(code)).decode()
        raise RuntimeError(f"{what} failed: {msg} (code {code})")
    return code


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODES[dtype]
    except KeyError:
        raise TypeError(f"castle HIP kernels support float32, bfloat16 and float16, not {dtype}") from None


def view4(t: torch.Tensor) -> View4:
    """castle_view4 of a (B, H, L, d) tensor with unit stride along d."""
    assert t.dim() == 4 and (t.stride(3) == 1 or t.shape[3] == 1)
    return View4(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def vector_ok(t: torch.Tensor) -> bool:
    """True if the kernels can read `t` in place: unit stride along d, 16-byte aligned rows."""
    q = 16 // t.element_size()
    return (
        t.stride(3) == 1
        and t.data_ptr() % 16 == 0
        and all(t.stride(i) % q == 0 for i in range(3))
    )


def stream_ptr(device) -> int:
    return torch.cuda.current_stream(device).cuda_stream


PROFILE_SLOTS = ("prep", "scan", "attn", "delta", "bwd_key", "bwd_query", "decode_stream", "decode_finish")


def profile_enable(on: bool):
    check(lib().castle_profile_enable(1 if on else 0), "castle_profile_enable")


def profile_read(max_records: int = 65536):
    """[(slot name, milliseconds), ...] of the kernels launched since profiling was enabled."""
    slots = (ctypes.c_int * max_records)()
    ms = (ctypes.c_float * max_records)()
    n = check(lib().castle_profile_read(slots, ms, max_records), "castle_profile_read")
    return [(PROFILE_SLOTS[slots[i]], ms[i]) for i in range(n)]
