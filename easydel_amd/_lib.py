"""ctypes binding of librpa_hip.so (the C ABI declared in include/rpa_hip.h and include/rpa_hip_probe.h).

There is no fallback: if the library is missing or fails to load, every call raises.
"""

from __future__ import annotations

import ctypes
import threading
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "librpa_hip.so"

# rpa_dtype tags
RPA_F32, RPA_BF16, RPA_FP8_E4M3, RPA_INT8, RPA_F16 = 0, 1, 2, 3, 4
RPA_ERR_INVALID_ARGUMENT, RPA_ERR_UNSUPPORTED, RPA_ERR_WORKSPACE = -1, -2, -3

_c_int, _c_i64, _c_f32, _c_vp, _c_sz = ctypes.c_int, ctypes.c_int64, ctypes.c_float, ctypes.c_void_p, ctypes.c_size_t

# name -> (restype, argtypes); mirrors the two headers declaration by declaration.
SIGNATURES = {
    "rpa_version": (ctypes.c_char_p, []),
    "rpa_last_error": (ctypes.c_char_p, []),
    "rpa_set_tunable": (_c_int, [ctypes.c_char_p, _c_int]),
    "rpa_page_scatter_slices": (_c_int, [_c_vp, _c_vp, _c_vp, _c_vp, _c_vp, _c_int, _c_int, _c_i64, _c_int, _c_i64, _c_int]),
    "rpa_page_scatter_ragged": (_c_int, [_c_vp] * 8 + [_c_int] * 10),
    "rpa_attention_workspace_bytes": (_c_sz, [_c_int] * 9),
    "rpa_ragged_paged_attention": (
        _c_int,
        [_c_vp] * 10 + [_c_sz] + [_c_int] * 12 + [_c_f32, _c_int, _c_f32, _c_vp],
    ),
    "rpa_page_scatter_ragged_quantised": (_c_int, [_c_vp] * 9 + [_c_int] * 11),
    "rpa_ragged_paged_attention_v3_quantised": (
        _c_int,
        [_c_vp] * 12 + [_c_sz] + [_c_int] * 13 + [_c_f32, _c_int, _c_f32, _c_vp],
    ),
    "rpa_unified_attention": (
        _c_int,
        [_c_vp] * 11 + [_c_sz] + [_c_int] * 10 + [_c_f32, _c_int, _c_f32, _c_vp],
    ),
    "rpa_ragged_paged_attention_v3": (
        _c_int,
        [_c_vp] * 11 + [_c_sz] + [_c_int] * 12 + [_c_f32, _c_int, _c_f32, _c_vp],
    ),
    "rpa_ragged_paged_attention_v3_static": (
        _c_int,
        [_c_vp] * 10 + [_c_int] * 12 + [_c_f32, _c_int, _c_f32, _c_vp],
    ),
    "rpa_mla_ragged_paged_attention": (
        _c_int,
        [_c_vp] * 12 + [_c_sz] + [_c_int] * 11 + [_c_f32, _c_int, _c_f32, _c_vp],
    ),
    "rpa_mla_workspace_bytes": (_c_sz, [_c_int] * 8),
    "rpa_mla_page_scatter": (_c_int, [_c_vp] * 8 + [_c_int] * 9),
}


# the measurement kernels of rpa_hip_probe.h: exported by the test / benchmark build of the library only
PROBE_SIGNATURES = {
    "rpa_calibration_copy": (_c_int, [_c_vp, _c_vp, _c_vp, _c_sz]),
    "rpa_read_probe": (_c_sz, [_c_vp, _c_vp, _c_sz, _c_int, _c_int, _c_vp]),
    "rpa_read_probe_paged": (_c_sz, [_c_vp, _c_vp, _c_sz, _c_int, _c_int, _c_int, _c_int, _c_vp]),
    "rpa_mfma_probe": (ctypes.c_double, [_c_vp, _c_int, _c_int, _c_int, _c_int, _c_int, _c_vp, _c_vp]),
    "rpa_issue_probe": (ctypes.c_longlong, [_c_vp, _c_int, _c_int, _c_int, _c_int, _c_vp, _c_vp, _c_vp]),
}


class RpaError(RuntimeError):
    """A C-ABI call returned non-zero."""

    def __init__(self, code: int, message: str):
        super().__init__(f"librpa_hip error {code}: {message}")
        self.code = code


_lock = threading.Lock()
_lib = None


def load() -> ctypes.CDLL:
    """Load the library once and attach prototypes.  Raises if it has not been built."""
    global _lib
    with _lock:
        if _lib is None:
            if not LIB_PATH.exists():
                raise RuntimeError(
                    f"{LIB_PATH} is missing: build it with `python -m easydel_amd.build` "
                    "(there is no CPU or PyTorch fallback for this path)"
                )
            # PyTorch owns the device memory and streams this library is handed, so its HIP runtime must be the one
            # in the process: loaded first here, the system's copy of the runtime would take its place and the
            # library's first launch would find no device.
            import torch  # noqa: F401

            lib = ctypes.CDLL(str(LIB_PATH))
            for name, (restype, argtypes) in SIGNATURES.items():
                fn = getattr(lib, name)
                fn.restype = restype
                fn.argtypes = argtypes
            for name, (restype, argtypes) in PROBE_SIGNATURES.items():
                fn = getattr(lib, name, None)  # absent from a product build
                if fn is not None:
                    fn.restype = restype
                    fn.argtypes = argtypes
            _lib = lib
    return _lib


def check(code: int) -> None:
    if code != 0:
        raise RpaError(code, load().rpa_last_error().decode("utf-8", "replace"))


def set_tunable(name: str, value: int) -> int:
    return int(load().rpa_set_tunable(name.encode(), int(value)))
