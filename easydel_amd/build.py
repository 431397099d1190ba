"""Builds librpa_hip.so (hand-written HIP kernels + C ABI) for gfx950 with hipcc.

Run as ``python -m easydel_amd.build``; hipcc cross-compiles without a GPU.  The library is
written next to the package (``easydel_amd/lib/librpa_hip.so``) so it travels with the tree.
"""

from __future__ import annotations

import concurrent.futures
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OUT_DIR = PKG / "lib"
LIB_PATH = OUT_DIR / "librpa_hip.so"

SOURCES = [
    "rpa_api.hip",
    "rpa_scatter.hip",
    "rpa_attn_generic.hip",
    "rpa_attn_decode.hip",
    "rpa_attn_prefill.hip",
    "rpa_attn_prefill_dma.hip",
    "rpa_attn_prefill_dma8.hip",
    "rpa_attn_prefill_x32.hip",
    "rpa_widen.hip",
    "rpa_attn_merge.hip",
    "rpa_mla.hip",
]
# measurement kernels and result-changing test knobs: compiled into the test / benchmark build only (-DRPA_PROBES)
PROBE_SOURCES = ["rpa_probe.hip"]

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 from scalar float code on this target.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the HIP library cannot be built")
    return exe


def _compile(src: str, obj_dir: Path, extra: list[str]) -> Path:
    obj = obj_dir / (Path(src).stem + ".o")
    cmd = [_hipcc(), *HIPCC_FLAGS, *extra, "-c", str(CSRC / src), "-o", str(obj)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{res.stderr[-6000:]}")
    return obj


def build_library(verbose: bool = True, extra_flags: list[str] | None = None, jobs: int = 6, probes: bool = True) -> Path:
    """Compile every kernel source and link the shared library.  Always rebuilds.  ``probes=False`` is the product
    build: no measurement kernels, and ``rpa_set_tunable`` does not know the knobs that can make a call skip a stage."""
    extra = list(extra_flags or []) + (["-DRPA_PROBES"] if probes else [])
    sources = SOURCES + (PROBE_SOURCES if probes else [])
    obj_dir = OUT_DIR / "obj"
    obj_dir.mkdir(parents=True, exist_ok=True)
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, obj_dir, extra), sources))
    tmp = LIB_PATH.with_suffix(".so.tmp")
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", *map(str, objs), "-o", str(tmp)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr[-4000:]}")
    os.replace(tmp, LIB_PATH)
    if verbose:
        print(f"built {LIB_PATH} ({LIB_PATH.stat().st_size} bytes)")
    return LIB_PATH


def build_ffi(verbose: bool = True) -> Path | None:
    """Compile csrc/rpa_ffi.cc (the XLA FFI handlers over the C ABI) into lib/librpa_ffi.so.  It needs jaxlib's
    ``xla/ffi/api`` headers: where ``jax.ffi`` does not import, nothing is built and None is returned."""
    try:
        import jax.ffi as jax_ffi
    except Exception:  # jax is not installed on this host
        if verbose:
            print("jax.ffi is not importable here: librpa_ffi.so is not built")
        return None
    out = OUT_DIR / "librpa_ffi.so"
    cmd = [_hipcc(), "-shared", "-fPIC", "-std=c++17", "-O2", f"-I{jax_ffi.include_dir()}", str(CSRC / "rpa_ffi.cc"),
           f"-L{OUT_DIR}", "-lrpa_hip", "-Wl,-rpath,$ORIGIN", "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on rpa_ffi.cc:\n{res.stderr[-6000:]}")
    if verbose:
        print(f"built {out}")
    return out


if __name__ == "__main__":
    args = sys.argv[1:]
    product = "--product" in args
    build_library(extra_flags=[a for a in args if a != "--product"], probes=not product)
    build_ffi()
