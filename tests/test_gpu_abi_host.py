"""The C ABI without Python or PyTorch in the process: a C++ program (tests/abi_host.cpp, built by
``__graft_entry__.build()``) dlopens librpa_hip.so, allocates with hipMalloc and runs the golden float32 batch."""

import os
import struct
import subprocess

import numpy as np
import pytest

from easydel_amd import _lib

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))


def test_c_abi_from_a_plain_cpp_host(gpu, tmp_path):
    exe = os.path.join(HERE, "abi_host")
    assert os.path.exists(exe), "tests/abi_host is missing: build it with `python __graft_entry__.py`"
    z = np.load(os.path.join(HERE, "golden", "attention_c1_fp32.npz"))
    q, bt = z["query"], z["block_tables"]
    T, Hq, D = q.shape
    S, M = bt.shape
    P, pg, C = int(z["num_pages"]), z["live_page_values"].shape[1], z["live_page_values"].shape[2]
    pages = np.zeros((P, pg, C, D), np.float32)
    pages[z["live_pages"]] = z["live_page_values"]
    path = tmp_path / "c1.bin"
    with open(path, "wb") as f:
        f.write(struct.pack("<9i", 0x52504131, T, S, M, P, pg, Hq, C // 2, D))
        f.write(struct.pack("<f", float(z["softmax_scale"])))
        for a, dt in ((q, np.float32), (pages, np.float32), (z["context_lens"], np.int32), (bt, np.int32),
                      (z["query_start_loc"], np.int32), (z["num_seqs"], np.int32), (z["expected"], np.float32)):
            f.write(np.ascontiguousarray(a, dtype=dt).tobytes())
    res = subprocess.run([exe, str(_lib.LIB_PATH), str(path)], capture_output=True, text=True, timeout=120)
    print(res.stdout, res.stderr, flush=True)
    assert res.returncode == 0 and res.stdout.strip().endswith("abi_host OK"), (res.returncode, res.stdout, res.stderr)
    assert res.stdout.count(" ok") == 4  # float32 and bf16, read-only and fused
