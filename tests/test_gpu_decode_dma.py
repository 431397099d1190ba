"""GPU parity of the LDS-direct decode kernel (tiles moved global -> LDS by the load unit, two tiles in flight per wave,
its own waits): against the oracle, and bit for bit against the register-staged decode kernel, which does the same
arithmetic in the same order.  By default a call uses it for head size 256 only; the knob routes every shape it is
built for through it."""

import numpy as np
import pytest

import rpa_testlib as tl
from easydel_amd import _lib
from rpa_testlib import BF16, FP8, INT8

pytestmark = pytest.mark.gpu


def _both(b, **kw):
    prev = _lib.set_tunable("decode_dma", 0)
    try:
        staged = tl.run_gpu_attention(b, **kw)
        _lib.set_tunable("decode_dma", 1)
        direct = tl.run_gpu_attention(b, **kw)
        _lib.set_tunable("decode_dma", 3)  # the K rows of a tile requested together with its V rows
        other = tl.run_gpu_attention(b, **kw)
        assert np.array_equal(other[tl.valid_rows(b)], direct[tl.valid_rows(b)]), "decode_dma 3 differs"
    finally:
        _lib.set_tunable("decode_dma", prev)
    return staged, direct


CASES = [
    # kv dtype, D, Hq, Hkv, page size
    (BF16, 128, 32, 8, 64),
    (BF16, 128, 16, 4, 128),
    (BF16, 64, 64, 8, 64),
    (BF16, 256, 16, 8, 64),
    (FP8, 128, 40, 8, 64),
    (INT8, 128, 40, 8, 64),
    (FP8, 128, 32, 8, 128),
]


@pytest.mark.parametrize("kv_dtype,D,Hq,Hkv,page_size", CASES)
def test_lds_direct_decode_matches_oracle_and_register_kernel(gpu, kv_dtype, D, Hq, Hkv, page_size):
    """Decode rows and short multi-token rows over contexts from one key to a few thousand (several pages, page
    boundaries inside tiles, contexts that end inside a tile), padded rows and tokens; then with a window whose left
    edge falls inside a tile and a soft cap; then cut into many spans so that rows are merged from partial slots."""
    ctx = [1, 17, 64, 65, 700, 2049, 3000, 129, 4095, 31, 900, 1024]
    q = [1, 1, 1, 2, 1, 3, 1, 1, 1, 1, 2, 1]
    b = tl.make_batch(900 + D + page_size + kv_dtype, ctx, q, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype,
                      pad_rows=2, pad_tokens=3)
    if kv_dtype == FP8:  # slots past each context hold NaN codes: nobody may read them as data
        for i, c in enumerate(b.context_lens[:b.n]):
            if c % page_size:
                b.kv_raw[b.block_tables[i, c // page_size], c % page_size:] = 0x7F
    above_4 = kv_dtype != BF16  # scaled codes: rows that see one or two keys return values beyond 4
    for kw in ({}, dict(sliding_window=777, logits_soft_cap=30.0)):
        staged, direct = _both(b, **kw)
        tl.assert_close(direct, tl.oracle_out(b, **kw), b, f"LDS-direct decode kv{kv_dtype} D{D} {sorted(kw)}", one_ulp_above_4=above_4)
        assert np.array_equal(direct[tl.valid_rows(b)], staged[tl.valid_rows(b)]), "the two decode kernels differ"
    prev = _lib.set_tunable("decode_wgs", 37)
    try:
        staged, direct = _both(b)
    finally:
        _lib.set_tunable("decode_wgs", prev)
    tl.assert_close(direct, tl.oracle_out(b), b, "LDS-direct decode, 37 spans", one_ulp_above_4=above_4)
    assert np.array_equal(direct[tl.valid_rows(b)], staged[tl.valid_rows(b)])


def test_lds_direct_decode_unscaled_fp8(gpu):
    b = tl.make_batch(977, [700, 65, 1500, 300, 33], [1, 1, 2, 1, 1], Hq=40, Hkv=8, D=128, page_size=64, kv_dtype=FP8, scaled=False)
    staged, direct = _both(b)
    tl.assert_close(direct, tl.oracle_out(b), b, "LDS-direct decode, unscaled fp8")
    assert np.array_equal(direct[tl.valid_rows(b)], staged[tl.valid_rows(b)])
