"""Pins the C restatement (the cpu_baseline leg's code) against the float64 numpy oracle."""

import numpy as np
import pytest

import rpa_testlib as tl
from oracle import c_oracle
from rpa_testlib import BF16, F32, FP8, INT8, orc


@pytest.fixture(scope="module", autouse=True)
def _built():
    if not c_oracle.LIB.exists():
        c_oracle.build()


@pytest.mark.parametrize("q_dtype,kv_dtype", [(F32, F32), (BF16, BF16), (BF16, FP8), (BF16, INT8), (F32, BF16)])
@pytest.mark.parametrize("kw", [{}, {"sliding_window": 40}, {"logits_soft_cap": 5.0, "softmax_scale": 0.2}])
def test_c_oracle_matches_numpy_oracle(q_dtype, kv_dtype, kw):
    b = tl.make_batch(31, [17, 64, 130, 255, 1], [1, 1, 8, 33, 1], Hq=8, Hkv=2, D=64, page_size=16, q_dtype=q_dtype,
                      kv_dtype=kv_dtype, pad_rows=2, pad_tokens=3)
    want = tl.oracle_out(b, **kw)
    got = c_oracle.attention(b.q_raw, q_dtype, b.kv_raw, kv_dtype, b.kv_scales, b.context_lens, b.block_tables,
                             b.query_start_loc, b.num_seqs, Hkv=b.Hkv, num_threads=2, **kw)
    assert np.abs(got - want).max() <= 1e-5
    assert np.all(got[int(b.query_start_loc[b.n]):] == 0)


def test_c_scatter_matches_numpy_oracle():
    import ctypes

    b = tl.make_batch(32, [17, 64, 130], [1, 8, 33], Hq=2, Hkv=2, D=8, page_size=16, kv_dtype=BF16)
    rng = np.random.default_rng(0)
    key = rng.integers(0, 65535, size=(b.T, 2, 8), dtype=np.uint16)
    val = rng.integers(0, 65535, size=(b.T, 2, 8), dtype=np.uint16)
    want = orc.page_scatter_ragged_ref(key, val, b.kv_raw, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
    pages = b.kv_raw.copy()
    lib = c_oracle.load()
    p = lambda a: a.ctypes.data_as(ctypes.c_void_p)
    bt = np.ascontiguousarray(b.block_tables)
    lib.rpa_oracle_scatter_ragged(p(key), p(val), p(pages), p(b.context_lens), p(bt), p(b.query_start_loc), 3, b.M, 16, 2, 8, 4, 2)
    np.testing.assert_array_equal(pages, want)
