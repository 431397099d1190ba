"""GPU parity of float16 queries over float16 pages on the MFMA kernels (half-precision operands, float32 accumulation):
the decode kernels (register-staged and LDS-direct), the LDS-direct prefill kernel and the merge of split rows,
against the oracle and against the float32 kernel on the same inputs.  Other float16 combinations (mixed with bf16 or
float32, page sizes that are not a multiple of 32) stay on the float32 kernel (tests/test_gpu_formats.py)."""

import numpy as np
import pytest

import rpa_testlib as tl
from easydel_amd import _lib
from rpa_testlib import F16

pytestmark = pytest.mark.gpu


def _mfma_and_fp32(b, **kw):
    got = tl.run_gpu_attention(b, **kw)
    prev = _lib.set_tunable("force_generic", 1)
    try:
        slow = tl.run_gpu_attention(b, **kw)
    finally:
        _lib.set_tunable("force_generic", prev)
    return got, slow


@pytest.mark.parametrize("D,Hq,Hkv,page_size", [(128, 32, 8, 64), (64, 16, 2, 32), (256, 16, 8, 128), (128, 8, 1, 64)])
def test_float16_decode_and_prefill_on_the_mfma_kernels(gpu, D, Hq, Hkv, page_size):
    ctx = [1, 17, 64, 65, 700, 2049, 3000, 129, 900, 5000]
    q = [1, 1, 1, 2, 1, 3, 300, 129, 33, 520]
    b = tl.make_batch(1200 + D + page_size, ctx, q, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, q_dtype=F16, kv_dtype=F16,
                      pad_rows=1, pad_tokens=3)
    for kw in ({}, dict(sliding_window=777, logits_soft_cap=30.0)):
        got, slow = _mfma_and_fp32(b, **kw)
        want = tl.oracle_out(b, **kw)
        mx, mean = tl.assert_close(got, want, b, f"float16 MFMA D{D} pg{page_size} {sorted(kw)}")
        print(f"float16 MFMA D{D} pg{page_size} {sorted(kw)}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
        tl.assert_close(slow, want, b, "float16 on the float32 kernel")
        assert not np.array_equal(got, slow), "the MFMA kernels did not run"
    assert np.all(got[int(b.query_start_loc[b.n]):] == 0.0), "padded token rows must be written as zeros"


def test_float16_split_rows_sinks_and_lds_direct_decode(gpu):
    """Decode rows merged from many spans, prefill row tiles split over key chunks, attention sinks, and the LDS-direct
    decode kernel, bit-identical to the register-staged one."""
    b = tl.make_batch(1290, [9000, 4100, 700, 64, 12000], [1, 2, 1, 1, 200], Hq=32, Hkv=8, D=128, page_size=64, q_dtype=F16, kv_dtype=F16)
    sinks = np.linspace(-2.0, 3.0, b.Hq).astype(np.float32)
    prev = (_lib.set_tunable("decode_wgs", 23), _lib.set_tunable("prefill_chunks", 4))
    try:
        got = tl.run_gpu_attention(b, softmax_aux=sinks)
        tl.assert_close(got, tl.oracle_out(b, softmax_aux=sinks), b, "float16, split rows, sinks")
        old = _lib.set_tunable("decode_dma", 1)
        try:
            direct = tl.run_gpu_attention(b, softmax_aux=sinks)
        finally:
            _lib.set_tunable("decode_dma", old)
        assert np.array_equal(direct[tl.valid_rows(b)], got[tl.valid_rows(b)])
    finally:
        _lib.set_tunable("decode_wgs", prev[0])
        _lib.set_tunable("prefill_chunks", prev[1])
