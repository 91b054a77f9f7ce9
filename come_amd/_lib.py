"""ctypes binding of ``libcome_hip.so`` (the C ABI declared in ``include/come_hip.h``).

There is no fallback: if the library has not been built, loading raises and every
operator of this package is unusable.  Build it with ``python -m come_amd.build``.
"""

from __future__ import annotations

import ctypes
import os
import threading

import torch  # noqa: F401  (imported first so the process binds one HIP runtime, torch's)

_HERE = os.path.dirname(os.path.abspath(__file__))
# COME_HIP_LIBRARY points at an alternative build of the same library (e.g. an experimental variant)
LIB_PATH = os.environ.get("COME_HIP_LIBRARY") or os.path.join(_HERE, "lib", "libcome_hip.so")

COME_F32, COME_F16, COME_BF16 = 0, 1, 2
COME_ATTN_FOLD_SCALE, COME_ATTN_WORK_QUEUE = 1, 2          # bits of the attention entry points' `flags`

_DTYPE_CODE = {torch.float32: COME_F32, torch.float16: COME_F16, torch.bfloat16: COME_BF16}

_i64 = ctypes.c_int64
_ptr = ctypes.c_void_p
_int = ctypes.c_int
_f32 = ctypes.c_float



class QPrologue(ctypes.Structure):
    """``come_q_prologue`` of the header: the q-side arguments of ``come_qk_norm_rope`` for ``come_attn_varlen_fwd_qp``."""
    _fields_ = [("apply_norm", _int), ("eps", _f32), ("weight", _ptr), ("bias", _ptr), ("positions", _ptr),
                ("cos_table", _ptr), ("sin_table", _ptr), ("n_pos", _i64)]


# name -> (restype, argtypes); must list every function declared in include/come_hip.h
SIGNATURES = {
    "come_version": (_int, []),
    "come_last_error": (ctypes.c_char_p, []),
    "come_merge_plan": (_int, [_ptr, _i64, _i64, _i64, _i64, _i64, _ptr, _ptr, _ptr]),
    "come_token_merge": (_int, [_ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr]),
    "come_token_split": (_int, [_ptr, _int, _i64, _i64, _ptr, _ptr, _i64, _ptr, _ptr]),
    "come_token_split_pair": (_int, [_ptr, _ptr, _int, _i64, _i64, _ptr, _ptr, _i64, _ptr, _ptr]),
    "come_select_windows": (_int, [_ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64, _int, _f32,
                                   _ptr, _ptr, _ptr, _i64, _ptr]),
    "come_select_plan": (_int, [_ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64, _int, _f32, _i64,
                                _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr]),
    "come_select_work_bytes": (_i64, [_i64, _i64, _i64, _i64, _i64, _i64]),
    "come_attn_varlen_fwd": (_int, [_ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64,
                                    _ptr, _i64, _i64, _i64, _i64, _ptr, _i64, _f32,
                                    _ptr, _i64, _i64, _ptr, _int, _ptr]),
    "come_attn_work_bytes": (_i64, [_i64, _i64, _i64, _i64]),
    "come_attn_queue_bytes": (_i64, [_i64, _i64, _i64]),
    "come_attn_varlen_fwd_ws": (_int, [_ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64,
                                       _ptr, _i64, _i64, _i64, _i64, _ptr, _i64, _f32,
                                       _ptr, _i64, _i64, _ptr, _ptr, _i64, _int, _ptr]),
    "come_attn_varlen_fwd_qp": (_int, [_ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64,
                                       _ptr, _i64, _i64, _i64, _i64, _ptr, _i64, _f32,
                                       _ptr, _i64, _i64, _ptr, _ptr, _i64, ctypes.POINTER(QPrologue), _int, _ptr]),
    "come_attn_static_work_bytes": (_i64, []),
    "come_attn_varlen_fwd_static": (_int, [_ptr, _ptr, _ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64,
                                           _ptr, _i64, _i64, _i64, _i64, _ptr, _i64, _f32,
                                           _ptr, _i64, _i64, _ptr, _int, _ptr]),
    "come_qk_norm_rope": (_int, [_ptr, _ptr, _int, _i64, _i64, _i64, _i64, _i64, _i64, _i64,
                                 _int, _ptr, _ptr, _ptr, _ptr, _f32, _ptr, _ptr, _ptr, _i64, _ptr]),
    "come_jagged_add_suffix": (_int, [_ptr, _ptr, _int, _i64, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr]),
    "come_jagged_split_suffix": (_int, [_ptr, _ptr, _int, _i64, _i64, _ptr, _i64, _i64, _ptr, _ptr, _ptr, _ptr,
                                        _ptr]),
}

_lock = threading.Lock()
_lib = None


def load() -> ctypes.CDLL:
    """Returns the loaded library, loading it on first use."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            if not os.path.exists(LIB_PATH):
                raise RuntimeError(
                    f"{LIB_PATH} is missing: the HIP library of come_amd has not been built "
                    "(run `python -m come_amd.build`). There is no fallback implementation."
                )
            lib = ctypes.CDLL(LIB_PATH)
            lib.come_version.restype = ctypes.c_int
            if lib.come_version() < 201:
                raise RuntimeError(f"{LIB_PATH} is an older build of libcome_hip (version {lib.come_version()}, this "
                                   "binding needs 0.2.1: `flags` on the attention entry points, "
                                   "come_attn_varlen_fwd_qp); rebuild with `python -m come_amd.build`")
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            _lib = lib
    return _lib


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return _DTYPE_CODE[dtype]
    except KeyError:
        raise RuntimeError(f"come_amd: unsupported dtype {dtype} (float32, float16, bfloat16 only)") from None


def check(status: int) -> None:
    """Turns a non-zero status of the C ABI into ``RuntimeError`` (as TORCH_CHECK does in the reference)."""
    if status != 0:
        msg = load().come_last_error().decode("utf-8", "replace")
        raise RuntimeError(msg or f"libcome_hip call failed with status {status}")


def ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


_RAW_STREAM = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream(device: torch.device) -> int:
    """Handle of torch's current HIP stream on ``device`` (the raw getter skips building a Stream object)."""
    if _RAW_STREAM is not None:
        return _RAW_STREAM(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


def require_gpu_tensor(t: torch.Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be on the GPU (got device {t.device})")
