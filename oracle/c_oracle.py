"""ctypes loader for the C restatement (oracle/rpa_oracle_c.c).  TEST INFRASTRUCTURE ONLY.

Used by tests/test_oracle_c.py (pins it against the numpy oracle) and by bench.py's cpu_baseline leg.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "lib" / "librpa_oracle.so"


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-B", "lib/librpa_oracle.so"], check=True, capture_output=True)
    return LIB


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not LIB.exists():
            raise RuntimeError(f"{LIB} missing: run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(str(LIB))
        vp, i32, f32 = ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        lib.rpa_oracle_attention.restype = i32
        lib.rpa_oracle_attention.argtypes = [vp, i32, vp, i32, vp, vp, vp, vp, i32, vp] + [i32] * 9 + [f32, i32, f32, i32]
        lib.rpa_oracle_scatter_ragged.restype = None
        lib.rpa_oracle_scatter_ragged.argtypes = [vp] * 6 + [i32] * 7
        lib.rpa_oracle_max_threads.restype = i32
        _lib = lib
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def attention(q_raw, q_dtype, kv_raw, kv_dtype, kv_scales, context_lens, block_tables, qsl, num_seqs, *, Hkv,
              softmax_scale=None, sliding_window=None, logits_soft_cap=None, num_threads=0) -> np.ndarray:
    """Raw storage arrays in, float32 [T, Hq, D] out."""
    lib = load()
    T, Hq, D = q_raw.shape
    P, pg, C = kv_raw.shape[0], kv_raw.shape[1], kv_raw.shape[2]
    S = len(context_lens)
    bt = np.ascontiguousarray(block_tables, dtype=np.int32).reshape(S, -1)
    out = np.empty((T, Hq, D), dtype=np.float32)
    scale = float(D) ** -0.5 if softmax_scale is None else float(softmax_scale)
    q_raw, kv_raw = np.ascontiguousarray(q_raw), np.ascontiguousarray(kv_raw)
    ctx = np.ascontiguousarray(context_lens, dtype=np.int32)
    qs = np.ascontiguousarray(qsl, dtype=np.int32)
    sc = None if kv_scales is None else np.ascontiguousarray(kv_scales, dtype=np.float32)
    rc = lib.rpa_oracle_attention(_ptr(q_raw), q_dtype, _ptr(kv_raw), kv_dtype, _ptr(sc), _ptr(ctx), _ptr(bt), _ptr(qs),
                                  int(np.asarray(num_seqs).reshape(-1)[0]), _ptr(out), T, S, bt.shape[1], P, pg, Hq, Hkv, D, C,
                                  scale, int(sliding_window or 0), float(logits_soft_cap or 0.0), int(num_threads))
    if rc != 0:
        raise MemoryError("rpa_oracle_attention failed to allocate")
    return out


def max_threads() -> int:
    return int(load().rpa_oracle_max_threads())
