"""ctypes binding of ``libmlora_hip.so`` (C ABI declared in ``include/mlora.h``).

There is no fallback: if the shared library is missing or fails to load, importing
this module raises.  ``torch`` is imported first so that the HIP runtime PyTorch
ships is the one both sides use (the library only needs ``libamdhip64.so.7``).
"""
from __future__ import annotations

import ctypes as C
import os

import torch  # noqa: F401  (loads the HIP runtime before the extension)

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmlora_hip.so")
CSRC_DIR = os.path.normpath(os.path.join(_HERE, "..", "csrc"))

MLORA_OK = 0
MLORA_EINVAL, MLORA_ERANGE, MLORA_EALIGN, MLORA_EDTYPE, MLORA_ELAUNCH, MLORA_ENOSPACE = -1, -2, -3, -4, -5, -6
MLORA_F16, MLORA_BF16 = 0, 1
MAX_PROJ = 8
MAX_RANK = 64
GATHER_MAX_T = 8192
CNT_NSEG, CNT_NVALID, CNT_NCHUNK, CNT_BAD, CNT_WORDS = 0, 1, 2, 3, 8
WORK_WORDS = 80
SCATTER_MAX_JOBS = 16
NOALLOC_SCRATCH_BYTES = 16 << 20    # MLORA_NOALLOC_SCRATCH_BYTES


def work_cap(T: int) -> int:
    return ((T + 7) // 8) * 8


_vp, _i32, _i64, _f32 = C.c_void_p, C.c_int, C.c_int64, C.c_float

# name -> (restype, argtypes); one entry per function declared in include/mlora.h
SIGNATURES = {
    "mlora_last_error": (C.c_char_p, []),
    "mlora_version": (_i32, []),
    "mlora_pool_gather": (_i32, [_vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp,
                                 _vp, _vp, _vp, _i32, _vp, _vp, _vp]),
    "mlora_pool_scatter": (_i32, [_i32, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i64, _i32, _vp]),
    "mlora_host_alloc": (_i32, [_i64, _vp, _vp]),
    "mlora_host_free": (_i32, [_vp]),
    "mlora_assist_export": (_i32, [_vp, _i32, _i32, _i32, _vp, _i32, _i32, _vp, _i32, _i32, _i32, _i32, _i32, _vp]),
    "mlora_assist_import": (_i32, [_i32, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    "mlora_bgmv_workspace_bytes": (_i64, [_i32, _i32, _i32, _i32]),
    "mlora_bgmv_multi": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32,
                                _i64, _i32, _vp, _i32, _vp, _i64, _i32, _i32, _vp]),
    "mlora_bgmv_multi_noalloc": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32,
                                        _i64, _i32, _vp, _i32, _i32, _i32, _vp]),
    "mlora_bgmv": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i64,
                          _i32, _i32, _i32, _vp]),
    "mlora_bgmv_reflayout": (_i32, [_vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _f32, _i32, _vp]),
    "mlora_reflayout_plan_bytes": (_i64, [_i32]),
    "mlora_reflayout_plan": (_i32, [_vp, _i32, _i32, _i32, _i32, _i32, _vp, _i64, _vp]),
    "mlora_bgmv_reflayout_multi": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _f32, _i32,
                                          _i32, _i32, _vp, _i64, _vp]),
    "mlora_sgmv_workspace_bytes": (_i64, [_i32, _i32]),
    "mlora_sgmv": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                          _i32, _i64, _i32, _i32, _i32, _vp, _i64, _vp]),
    "mlora_sgmv_plan": (_i32, [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i64, _i32, _vp, _i64, _vp]),
    "mlora_sgmv_plan_aligned": (_i32, [_vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i64, _i32, _vp, _i64, _vp]),
    "mlora_sgmv_planned": (_i32, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32,
                                  _i32, _i64, _i32, _i32, _i32, _vp, _i64, _vp]),
    "mlora_sgmv_multi_workspace_bytes": (_i64, [_i32, _i32, _i32]),
    "mlora_sgmv_expand_cols": (_i32, [_i32, _i32, _i32, _i32]),
    "mlora_sgmv_multi_planned": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32,
                                        _i32, _i32, _i64, _i32, _i32, _i32, _vp, _i64, _vp]),
    "mlora_gemm_lora_planned": (_i32, [_i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _vp, _vp, _i32, _i32,
                                       _i32, _i32, _i64, _i32, _i32, _vp, _i64, _vp]),
    "mlora_prefill_reflayout": (_i32, [_vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp, _i64, _vp]),
}

_lib = None


class MloraError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"mlora error {code}: {message}")
        self.code = code


def lib() -> C.CDLL:
    """Load the extension (once).  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'` at the repository root)")
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)   # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


def check(rc: int) -> None:
    if rc != MLORA_OK:
        raise MloraError(rc, lib().mlora_last_error().decode("utf-8", "replace"))


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float16:
        return MLORA_F16
    if dt == torch.bfloat16:
        return MLORA_BF16
    raise TypeError(f"mlora kernels take float16 or bfloat16 tensors, got {dt}")


def ptr(t) -> int | None:
    """Device address of a tensor (None stays NULL)."""
    return None if t is None else t.data_ptr()


def current_stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream
