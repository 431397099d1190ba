"""GPU parity: HIP ragged paged attention (through the C ABI) against the float64 oracle."""

import numpy as np
import pytest

import rpa_testlib as tl
from rpa_testlib import BF16, F32, FP8, INT8

pytestmark = pytest.mark.gpu


def _check(b, what, **kw):
    got = tl.run_gpu_attention(b, **kw)
    want = tl.oracle_out(b, **kw)
    mx, mean = tl.assert_close(got, want, b, what)
    print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    return got


def test_config1_fp32_mixed_batch(gpu):
    # the tiny fp32 configuration: 4 sequences, ctx [17,64,130,255], q_lens [1,1,8,33], Hq 8, Hkv 2, D 64, page 16, 128 pages
    b = tl.make_batch(0, [17, 64, 130, 255], [1, 1, 8, 33], Hq=8, Hkv=2, D=64, page_size=16, num_pages=128,
                      q_dtype=F32, kv_dtype=F32)
    assert list(b.query_start_loc[:5]) == [0, 1, 2, 10, 43]
    _check(b, "C1 fp32", softmax_scale=1.0 / 8.0)


@pytest.mark.parametrize("D,page_size,Hq,Hkv", [(128, 64, 32, 8), (64, 16, 8, 2), (256, 128, 16, 8), (128, 16, 8, 1),
                                                 (128, 32, 24, 6), (64, 64, 32, 8)])
def test_bf16_decode(gpu, D, page_size, Hq, Hkv):
    rng = np.random.default_rng(D + page_size)
    ctx = rng.integers(1, 1600, size=12).tolist() + [1, 15, 16, 17, 512, 513, 1024]
    b = tl.make_batch(1, ctx, [1] * len(ctx), Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, max_pages=-(-1600 // page_size))
    _check(b, f"bf16 decode D{D} pg{page_size} Hq{Hq}/Hkv{Hkv}")


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
@pytest.mark.parametrize("D,page_size,Hq,Hkv", [(128, 64, 40, 8), (64, 16, 8, 2), (256, 32, 16, 8)])
def test_quantised_kv_decode(gpu, kv_dtype, D, page_size, Hq, Hkv):
    rng = np.random.default_rng(7)
    ctx = rng.integers(1, 1400, size=10).tolist() + [1, 31, 32, 33, 700]
    b = tl.make_batch(2, ctx, [1] * len(ctx), Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype,
                      max_pages=-(-1400 // page_size))
    _check(b, f"kv{kv_dtype} decode D{D} pg{page_size}")


def test_small_multi_token_rows(gpu):
    # speculative-style rows: q_len * group <= 16 stays on the split-K decode kernel with per-row causal limits
    ctx = [5, 64, 300, 1100, 777, 4, 2]
    q_lens = [4, 2, 3, 4, 1, 4, 2]
    b = tl.make_batch(3, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, max_pages=20)
    _check(b, "bf16 multi-token small rows")


@pytest.mark.parametrize("D,page_size,Hq,Hkv", [(128, 64, 32, 8), (64, 32, 64, 8), (128, 16, 40, 8), (64, 16, 16, 1)])
def test_multi_token_rows_of_17_to_32(gpu, D, page_size, Hq, Hkv):
    # speculative-decoding verification steps: 17..32 rows per KV head ride the decode kernel with two row blocks per
    # wave (bf16 pages, head size <= 128, a batch with more tokens than sequence rows); long contexts are cut into
    # spans and merged, every row has its own causal limit
    G = Hq // Hkv
    q_max = 32 // G
    ctx = [5, 64, 300, 1100, 777, 40, 33, 3000, 9]
    q_lens = [min(q, c) for q, c in zip([q_max, q_max - 1, q_max, 17 // G + 1, q_max, 1, q_max, q_max, q_max], ctx)]
    b = tl.make_batch(15 + D, ctx, q_lens, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, max_pages=-(-3000 // page_size))
    assert b.T > b.S and max(q * G for q in q_lens) > 16
    _check(b, f"bf16 rows up to 32, D{D} pg{page_size} {Hq}/{Hkv}")
    _check(b, f"bf16 rows up to 32 + window, D{D}", sliding_window=70)
    s = np.random.default_rng(D).uniform(-1.0, 6.0, size=Hq).astype(np.float32)
    got = tl.run_gpu_attention(b, softmax_aux=s, logits_soft_cap=30.0)
    tl.assert_close(got, tl.oracle_out(b, softmax_aux=s, logits_soft_cap=30.0), b, "rows up to 32 + sinks + soft cap")


def test_row_class_limit_follows_the_static_bounds(gpu):
    # the same sequences in a call whose bounds leave no room for multi-token rows (T <= S through padded sequence
    # rows) are served by the large-row kernel instead: both routes must agree with the oracle and with each other
    ctx = [300, 1100, 64, 2000]
    q_lens = [6, 8, 5, 7]
    wide = tl.make_batch(16, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, max_pages=32)
    padded = tl.make_batch(16, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, max_pages=32, pad_rows=40)
    assert wide.T > wide.S and padded.T <= padded.S
    a = _check(wide, "rows 20..32, decode kernel")
    c = _check(padded, "rows 20..32, large-row kernel")
    assert np.abs(a[tl.valid_rows(wide)] - c[tl.valid_rows(padded)]).max() <= 2e-2


@pytest.mark.parametrize("window", [1, 64, 100, 1000])
def test_sliding_window_decode(gpu, window):
    ctx = [1, window, window + 1, window + 2, 900, 1500, 65, 129]
    b = tl.make_batch(4, ctx, [1] * len(ctx), Hq=16, Hkv=4, D=128, page_size=64, max_pages=24)
    _check(b, f"bf16 window {window}", sliding_window=window)


def test_window_with_null_pages_left_of_window(gpu):
    # pages entirely left of the window are freed by the scheduler and their table entries become the null page
    # (page 0); poison page 0 with NaN bit patterns: it must never be read as data
    W, pg = 256, 64
    ctx = [1000, 1500, 700, 300]
    b = tl.make_batch(5, ctx, [1] * 4, Hq=16, Hkv=4, D=128, page_size=pg, max_pages=24)
    want = tl.oracle_out(b, sliding_window=W)
    for i, c in enumerate(ctx):
        first_needed = max(c - 1 - W + 1, 0) // pg
        b.block_tables[i, :first_needed] = 0
    b.kv_raw[0] = 0x7FC0  # bf16 NaN
    got = tl.run_gpu_attention(b, sliding_window=W)
    tl.assert_close(got, want, b, "window + null pages")


@pytest.mark.parametrize("cap", [50.0, 5.0])
def test_logit_soft_cap(gpu, cap):
    ctx = [3, 200, 1000, 64]
    b = tl.make_batch(6, ctx, [1, 1, 1, 1], Hq=16, Hkv=8, D=256, page_size=128, max_pages=8)
    _check(b, f"bf16 softcap {cap}", logits_soft_cap=cap, softmax_scale=1.0 / 16.0)
    bf = tl.make_batch(6, ctx, [1, 2, 5, 64], Hq=4, Hkv=2, D=64, page_size=16, q_dtype=F32, kv_dtype=F32)
    _check(bf, f"fp32 softcap {cap}", logits_soft_cap=cap)


def test_padding_rows_tokens_and_zero_length_rows(gpu):
    # padded sequence rows, padded tokens past qsl[num_seqs], and a live row index with q_len == 0
    ctx = [100, 0, 257, 64]
    q_lens = [1, 0, 1, 1]
    b = tl.make_batch(8, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, pad_rows=5, pad_tokens=7, max_pages=8)
    got = _check(b, "padding")
    assert np.all(got[int(b.query_start_loc[b.n]):] == 0.0), "padded token rows must be written as zeros"


def test_live_row_count_beyond_the_metadata_is_clamped(gpu):
    # a row count larger than the metadata arrays (a caller's mistake) must not index past them: it counts as "all rows"
    b = tl.make_batch(17, [100, 257, 64, 900], [1, 3, 1, 40], Hq=32, Hkv=8, D=128, page_size=64, max_pages=16)
    want = tl.oracle_out(b)
    b.num_seqs = np.array([b.S + 1000], dtype=np.int32)
    got = tl.run_gpu_attention(b)
    tl.assert_close(got, want, b, "row count beyond S")


def test_shared_prefix_pages(gpu):
    # prefix caching: the same physical pages appear in several block-table rows
    ctx = [640, 700, 1000, 650]
    b = tl.make_batch(9, ctx, [1] * 4, Hq=32, Hkv=8, D=128, page_size=64, shared_prefix_pages=9, max_pages=16)
    _check(b, "shared prefix")


def test_physical_page_permutation_is_bit_invariant(gpu):
    ctx = [333, 1200, 64, 2000]
    b = tl.make_batch(10, ctx, [1] * 4, Hq=32, Hkv=8, D=128, page_size=64, max_pages=32)
    got1 = tl.run_gpu_attention(b)
    rng = np.random.default_rng(0)
    perm = np.concatenate([[0], 1 + rng.permutation(b.P - 1)])  # new physical id of each page; null page stays
    kv2 = np.empty_like(b.kv_raw)
    kv2[perm] = b.kv_raw
    b.kv_raw = kv2
    b.block_tables = perm[b.block_tables].astype(np.int32)
    got2 = tl.run_gpu_attention(b)
    assert np.array_equal(got1[tl.valid_rows(b)], got2[tl.valid_rows(b)])


@pytest.mark.parametrize("q_dtype,kv_dtype", [(BF16, BF16), (F32, BF16), (BF16, F32), (BF16, FP8)])
def test_mixed_prefill_decode_batch(gpu, q_dtype, kv_dtype):
    ctx = [17, 64, 130, 255, 500, 33, 1]
    q_lens = [1, 1, 8, 33, 100, 33, 1]
    b = tl.make_batch(11, ctx, q_lens, Hq=8, Hkv=2, D=64, page_size=16, q_dtype=q_dtype, kv_dtype=kv_dtype)
    _check(b, f"mixed q{q_dtype} kv{kv_dtype}")


def test_mixed_batch_llama_shape(gpu):
    ctx = [1500, 900, 300, 40, 2048]
    q_lens = [1, 1, 256, 40, 130]
    b = tl.make_batch(12, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, max_pages=32)
    _check(b, "mixed llama-shaped")
    _check(b, "mixed llama-shaped window", sliding_window=200)


def test_generic_kernel_agrees_with_mfma_kernel(gpu):
    from easydel_amd import _lib

    ctx = [1500, 900, 300, 40, 2048, 1]
    b = tl.make_batch(13, ctx, [1] * 6, Hq=32, Hkv=8, D=128, page_size=64, max_pages=32)
    fast = tl.run_gpu_attention(b)
    prev = _lib.set_tunable("force_generic", 1)
    try:
        slow = tl.run_gpu_attention(b)
    finally:
        _lib.set_tunable("force_generic", prev)
    want = tl.oracle_out(b)
    tl.assert_close(slow, want, b, "generic")
    assert np.abs(fast - slow)[tl.valid_rows(b)].max() <= tl.TOL_BF16_MAX


@pytest.mark.parametrize("wgs,splits", [(1, 2), (3, 2), (7, 5), (64, 16), (1000, 64), (0, 0)])
def test_split_k_settings_do_not_change_results(gpu, wgs, splits):
    # the number of persistent workgroups and of partial slots decides where sequences are cut
    from easydel_amd import _lib

    ctx = [1, 63, 64, 65, 1000, 1999, 128]
    b = tl.make_batch(14, ctx, [1] * len(ctx), Hq=32, Hkv=8, D=128, page_size=64, max_pages=32)
    p1, p2 = _lib.set_tunable("decode_wgs", wgs), _lib.set_tunable("max_splits", splits)
    try:
        _check(b, f"wgs {wgs} splits {splits}")
    finally:
        _lib.set_tunable("decode_wgs", p1)
        _lib.set_tunable("max_splits", p2)


@pytest.mark.parametrize("D,page_size,Hq,Hkv,kv_dtype", [
    (128, 64, 32, 8, BF16), (64, 16, 8, 2, BF16), (256, 128, 16, 8, BF16), (128, 16, 40, 8, BF16),
    (128, 64, 40, 8, FP8), (128, 32, 8, 8, INT8), (256, 32, 16, 8, FP8), (64, 64, 32, 1, BF16), (64, 16, 4, 2, INT8)])
def test_prefill_mfma_kernel(gpu, D, page_size, Hq, Hkv, kv_dtype):
    # full prefill (prior context 0), chunked prefill deep into a context, ragged tile edges, one decode row
    ctx = [300, 1000, 129, 47, 2100, 700]
    q_lens = [300, 200, 129, 33, 17, 1]
    b = tl.make_batch(40 + D, ctx, q_lens, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype, pad_rows=2, pad_tokens=5)
    _check(b, f"prefill D{D} pg{page_size} {Hq}/{Hkv} kv{kv_dtype}")


@pytest.mark.parametrize("window", [1, 16, 100, 513])
def test_prefill_sliding_window(gpu, window):
    ctx = [600, 1500, window + 40, 64]
    q_lens = [600, 300, 40, 64]
    b = tl.make_batch(50, ctx, q_lens, Hq=16, Hkv=4, D=128, page_size=64, max_pages=24)
    _check(b, f"prefill window {window}", sliding_window=window)


def test_prefill_soft_cap_gemma_shape(gpu):
    ctx = [900, 2500]
    q_lens = [256, 200]
    b = tl.make_batch(51, ctx, q_lens, Hq=16, Hkv=8, D=256, page_size=128, max_pages=20)
    _check(b, "prefill softcap", logits_soft_cap=50.0, softmax_scale=1.0 / 16.0)
    _check(b, "prefill softcap + window", logits_soft_cap=50.0, softmax_scale=1.0 / 16.0, sliding_window=300)


def test_prefill_window_with_null_pages(gpu):
    W, pg = 200, 64
    ctx = [1500, 900]
    q_lens = [100, 64]
    b = tl.make_batch(52, ctx, q_lens, Hq=16, Hkv=4, D=128, page_size=pg, max_pages=24)
    want = tl.oracle_out(b, sliding_window=W)
    for i, (c, ql) in enumerate(zip(ctx, q_lens)):
        first_needed = max(c - ql - W + 1, 0) // pg
        b.block_tables[i, :first_needed] = 0
    b.kv_raw[0] = 0x7FC0
    got = tl.run_gpu_attention(b, sliding_window=W)
    tl.assert_close(got, want, b, "prefill window + null pages")


def test_prefill_window_with_null_pages_smaller_than_the_alignment(gpu):
    # 32-token pages: the 64-aligned start of the key range can fall on a page that lies wholly left of the window
    W, pg = 200, 32
    ctx = [1500, 900, 333]
    q_lens = [100, 64, 40]
    b = tl.make_batch(54, ctx, q_lens, Hq=16, Hkv=4, D=128, page_size=pg, max_pages=48)
    want = tl.oracle_out(b, sliding_window=W)
    for i, (c, ql) in enumerate(zip(ctx, q_lens)):
        first_needed = max(c - ql - W + 1, 0) // pg
        b.block_tables[i, :first_needed] = 0
    b.kv_raw[0] = 0x7FC0
    got = tl.run_gpu_attention(b, sliding_window=W)
    tl.assert_close(got, want, b, "prefill window + 32-token null pages")


@pytest.mark.parametrize("D,page_size", [(128, 64), (256, 128), (64, 32)])
def test_prefill_ignores_cache_slots_past_the_context(gpu, D, page_size):
    # slots of the last page beyond ctx hold NaN: they must never reach the accumulators, not even times zero
    ctx = [300, 1000, 129, 47, 2100]
    q_lens = [300, 200, 129, 33, 17]
    b = tl.make_batch(55, ctx, q_lens, Hq=16, Hkv=4, D=D, page_size=page_size)
    want = tl.oracle_out(b)
    for i, c in enumerate(ctx):
        if c % page_size:
            b.kv_raw[b.block_tables[i, c // page_size], c % page_size:] = 0x7FC0
    got = tl.run_gpu_attention(b)
    tl.assert_close(got, want, b, f"prefill with NaN past ctx D{D}")


@pytest.mark.parametrize("D,page_size,Hq,Hkv", [(128, 64, 32, 8), (256, 128, 16, 8), (64, 32, 8, 2)])
def test_prefill_register_staged_kernel_serves_bf16_too(gpu, D, page_size, Hq, Hkv):
    # bf16 pages normally take the kernel that loads tiles straight into LDS; the other one must agree
    from easydel_amd import _lib

    ctx = [300, 1000, 129, 47, 2100, 700]
    q_lens = [300, 200, 129, 33, 17, 1]
    b = tl.make_batch(56 + D, ctx, q_lens, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, pad_rows=2, pad_tokens=5)
    direct = _check(b, f"prefill D{D}, tiles loaded into LDS directly", sliding_window=700)
    prev = _lib.set_tunable("prefill_dma", 0)
    try:
        staged = _check(b, f"prefill D{D}, tiles staged through registers", sliding_window=700)
    finally:
        _lib.set_tunable("prefill_dma", prev)
    assert np.abs(direct[tl.valid_rows(b)] - staged[tl.valid_rows(b)]).max() <= 2e-2


@pytest.mark.parametrize("D,page_size,Hq,Hkv,cap", [(128, 64, 32, 8, None), (256, 128, 16, 8, 50.0), (256, 64, 8, 4, None)])
@pytest.mark.parametrize("window", [None, 333])
def test_prefill_kernel_on_32x32_tiles(gpu, D, page_size, Hq, Hkv, cap, window):
    # The large-row kernel built on 32x32x16 tiles (one workgroup per CU; 256 rows at head size 128, 128 at 256): contexts
    # that end on every residue of its 32-key blocks and make odd and even block counts, a chunk deep in a context, a row
    # tile with a single live row, key ranges cut into chunks by the device's rule and by a fixed count -- against the
    # oracle, and against the kernel on 16x16x32 tiles that serves these shapes when this one is switched off.
    from easydel_amd import _lib

    ctx = [1, 31, 32, 33, 95, 96, 97, 161, 640, 2100, 1500, 4000]
    q_lens = [1, 31, 32, 33, 95, 96, 97, 129, 640, 70, 513, 300]
    b = tl.make_batch(61 + D, ctx, q_lens, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, pad_rows=1, pad_tokens=3, max_pages=-(-4000 // page_size))
    kw = dict(sliding_window=window, logits_soft_cap=cap, softmax_scale=D ** -0.5)
    rows = tl.valid_rows(b)
    want = tl.oracle_out(b, **kw)

    def run(what):
        got = tl.run_gpu_attention(b, **kw)
        mx, mean = tl.assert_close(got, want, b, what)
        print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
        return got

    wide = run(f"32x32 prefill D{D} window {window}")
    for chunks in (3, 8):  # fixed chunk counts: every row tile of the long sequences leaves partials for the merge
        prev = _lib.set_tunable("prefill_chunks", chunks)
        try:
            cut = run(f"32x32 prefill D{D} window {window}, {chunks} key chunks")
        finally:
            _lib.set_tunable("prefill_chunks", prev)
        assert np.abs(cut[rows] - wide[rows]).max() <= 2e-2
    prev = _lib.set_tunable("prefill_x32", 0)
    try:
        narrow = run(f"16x16 prefill D{D} window {window}")
    finally:
        _lib.set_tunable("prefill_x32", prev)
    assert np.abs(wide[rows] - narrow[rows]).max() <= 2e-2
    again = tl.run_gpu_attention(b, **kw)
    assert np.array_equal(again[rows], wide[rows]), "two runs of the same call must agree bit for bit"


@pytest.mark.parametrize("D,page_size,Hq,Hkv,cap", [(128, 64, 32, 8, None), (256, 128, 16, 8, 50.0)])
@pytest.mark.parametrize("spread", [4, 16])
def test_prefill_holds_the_tolerance_on_peaked_scores(gpu, D, page_size, Hq, Hkv, cap, spread):
    # Scores with `spread` times the usual spread (sharply peaked rows, as trained heads produce them): an error in a score is
    # an error in the exponent of its weight, so whatever a kernel does to its queries ahead of the MFMAs shows here first.
    # (Queries scaled by the softmax scale and rounded back to bf16 read 3e-2 at spread 4 and 1.3e-1 at 16.)
    b = tl.make_batch(7 + D, [2100, 1500, 700], [640, 300, 700], Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, max_pages=-(-2100 // page_size))
    kw = dict(softmax_scale=spread * D ** -0.5, logits_soft_cap=cap)
    got = tl.run_gpu_attention(b, **kw)
    mx, mean = tl.assert_close(got, tl.oracle_out(b, **kw), b, f"peaked scores D{D} spread {spread}")
    print(f"peaked scores D{D} spread {spread}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)


@pytest.mark.parametrize("spread", [4, 16])
def test_decode_holds_the_tolerance_on_peaked_scores(gpu, spread):
    # the same for decode rows (the split-K decode kernel and the merge), with and without a soft cap
    for D, page_size, Hq, Hkv, cap in ((128, 64, 32, 8, None), (256, 128, 16, 8, 50.0)):
        b = tl.make_batch(11, [2100, 1500, 700, 4000, 33], [1, 1, 1, 1, 1], Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, max_pages=-(-4000 // page_size))
        kw = dict(softmax_scale=spread * D ** -0.5, logits_soft_cap=cap)
        tl.assert_close(tl.run_gpu_attention(b, **kw), tl.oracle_out(b, **kw), b, f"peaked scores, decode D{D} spread {spread}")


def test_chunked_prefill_equals_rows_of_single_shot_prefill(gpu):
    # the same keys, queried as one 384-token prefill and as its last 128-token chunk
    b_full = tl.make_batch(53, [384], [384], Hq=32, Hkv=8, D=128, page_size=64)
    full = tl.run_gpu_attention(b_full)
    b_chunk = tl.make_batch(53, [384], [128], Hq=32, Hkv=8, D=128, page_size=64)
    b_chunk.kv_raw, b_chunk.kv_val, b_chunk.block_tables = b_full.kv_raw, b_full.kv_val, b_full.block_tables
    b_chunk.q_raw, b_chunk.q_val = b_full.q_raw[256:], b_full.q_val[256:]
    chunk = tl.run_gpu_attention(b_chunk)
    assert np.abs(chunk - full[256:]).max() <= 2e-2
    tl.assert_close(chunk, tl.oracle_out(b_chunk), b_chunk, "chunk")


def test_single_long_sequence_spreads_over_many_workgroups(gpu):
    # one decode row over 70k keys: the key stream is cut into hundreds of pieces and merged in several rounds
    from easydel_amd import _lib

    b = tl.make_batch(70, [70_001], [1], Hq=32, Hkv=8, D=128, page_size=64)
    _check(b, "single long sequence")
    prev = _lib.set_tunable("max_splits", 256)
    try:
        _check(b, "single long sequence, 256 slots")
    finally:
        _lib.set_tunable("max_splits", prev)


def test_many_short_sequences(gpu):
    rng = np.random.default_rng(71)
    ctx = rng.integers(1, 200, size=1500).tolist()
    b = tl.make_batch(71, ctx, [1] * len(ctx), Hq=8, Hkv=2, D=64, page_size=16, pad_rows=48)
    _check(b, "1500 short sequences")


def test_more_sequences_than_one_look_up_round_covers(gpu):
    # 6 000 rows: the wave-wide sequence look-up needs a third round (64 * 64 < 6 000), the plan kernel's threads hold
    # several sequences each, and a few multi-token rows sit among the single tokens
    rng = np.random.default_rng(73)
    ctx = rng.integers(1, 60, size=6000)
    q = np.ones(6000, dtype=np.int64)
    for i in rng.choice(6000, size=40, replace=False):
        q[i] = int(rng.integers(1, min(int(ctx[i]), 9) + 1))
    b = tl.make_batch(73, ctx.tolist(), q.tolist(), Hq=8, Hkv=2, D=64, page_size=16, pad_rows=100, pad_tokens=7)
    _check(b, "6000 sequences")


def test_many_prompts_in_one_call(gpu):
    # 400 whole prompts and chunks of 17..150 tokens: row tiles of the large-row kernel found by slot among hundreds of
    # sequences, most tiles partly filled, single tokens in between
    rng = np.random.default_rng(74)
    q = rng.integers(17, 151, size=400)
    q[rng.choice(400, size=60, replace=False)] = 1
    ctx = q + rng.integers(0, 200, size=400) * (rng.random(400) < 0.5)
    b = tl.make_batch(74, ctx.tolist(), q.tolist(), Hq=8, Hkv=2, D=64, page_size=16, pad_rows=5, pad_tokens=3)
    _check(b, "400 prompts")
    _check(b, "400 prompts, window 50", sliding_window=50)


def test_hip_graph_replay_matches_eager(gpu):
    # the C ABI neither allocates nor synchronises, so a whole layer call can be captured and replayed
    import torch
    from easydel_amd import kernels

    b = tl.make_batch(72, [700, 65, 1500, 300, 2000], [1, 1, 2, 40, 1], Hq=32, Hkv=8, D=128, page_size=64, pad_rows=2)
    d = tl.device_batch(b, gpu)
    rng = np.random.default_rng(3)
    key = tl.to_torch(tl.orc.f32_to_bf16_bits(rng.standard_normal((b.T, 8, 128), dtype=np.float32)), BF16, gpu)
    val = tl.to_torch(tl.orc.f32_to_bf16_bits(rng.standard_normal((b.T, 8, 128), dtype=np.float32)), BF16, gpu)
    dist = torch.tensor([3, 5, 5], dtype=torch.int32, device=gpu)
    out = torch.empty_like(d["query"])

    def call():
        kernels.ragged_paged_attention_v3(d["query"], key, val, d["kv_pages"], d["context_lens"], d["block_tables"].reshape(-1),
                                          d["query_start_loc"], dist, out=out)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()  # warm-up on the capture stream: sizes the cached workspace outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    eager = out.clone()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call()
    for rep in range(4):
        out.zero_()
        d["query"].mul_(1.0)  # eager work between replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {rep} differs from the eager result"
    # new metadata in the same buffers is picked up by the next replay (nothing is baked in on the host)
    d["context_lens"][0] = 650
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    b.context_lens[0] = 650
    pages_after = tl.orc.page_scatter_ragged_ref(key.view(torch.int16).cpu().numpy().view(np.uint16), val.view(torch.int16).cpu().numpy().view(np.uint16),
                                                 d["kv_pages"].view(torch.int16).cpu().numpy().view(np.uint16), b.context_lens,
                                                 b.block_tables, b.query_start_loc, b.num_seqs)
    want = tl.oracle_out(b, kv_val=tl.orc.bf16_bits_to_f32(pages_after).astype(np.float64))
    tl.assert_close(tl.from_torch(out, BF16), want, b, "graph replay with new metadata")
