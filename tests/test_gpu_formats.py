"""GPU parity for the cache formats of the reference beyond plain bf16 / fp32 pages: the cast-only fp8 cache (no
scales), padded head storage (head sizes stored in rows of 128 / 256), float16, and query rows before position 0."""

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd import _lib, kernels
from easydel_amd.caching import RaggedPagesCacheConfig, RaggedPagesCacheView, RaggedPagesMetadata
from easydel_amd.operations import OperationMetadata, OperationRegistry
from rpa_testlib import BF16, F16, F32, FP8, orc

pytestmark = pytest.mark.gpu


def _check(b, what, above_4=False, **kw):
    got = tl.run_gpu_attention(b, **kw)
    mx, mean = tl.assert_close(got, tl.oracle_out(b, **kw), b, what, one_ulp_above_4=above_4)
    if tl.last_widened:
        print(f"  {tl.last_widened} element(s) with |want| >= 4 judged by one bf16 step instead of 2e-2", flush=True)
    print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    return got


# ---- fp8 pages without scales: the reference's own low-precision cache (a bare cast, scale 1) ------------------
@pytest.mark.parametrize("D,page_size,Hq,Hkv", [(128, 64, 32, 8), (64, 16, 8, 2), (256, 32, 8, 4)])
def test_unscaled_fp8_pages_decode_and_prefill(gpu, D, page_size, Hq, Hkv):
    b = tl.make_batch(300 + D, [700, 65, 1500, 300, 33], [1, 1, 2, 150, 33], Hq=Hq, Hkv=Hkv, D=D, page_size=page_size,
                      kv_dtype=FP8, scaled=False, pad_rows=1, pad_tokens=2)
    assert b.kv_scales is None
    got = _check(b, f"unscaled fp8 D{D}")
    # the same pages with scales of one give the same bits, and the fp32 kernel agrees within the tolerance
    b.kv_scales = np.ones((b.P, b.C), np.float32)
    assert np.array_equal(tl.run_gpu_attention(b), got)
    b.kv_scales = None
    prev = _lib.set_tunable("force_generic", 1)
    try:
        slow = tl.run_gpu_attention(b)
    finally:
        _lib.set_tunable("force_generic", prev)
    tl.assert_close(slow, tl.oracle_out(b), b, "unscaled fp8 on the fp32 kernel")


def _new_kv(rng, T, Hkv, D, tag):
    x = rng.standard_normal((2, T, Hkv, D), dtype=np.float32)
    if tag == BF16:
        raw = orc.f32_to_bf16_bits(x)
        return raw[0], raw[1], orc.bf16_bits_to_f32(raw).astype(np.float64)
    if tag == FP8:
        raw = orc.cast_e4m3fn_ref(x)
        return raw[0], raw[1], orc.e4m3fn_bits_to_f32(raw).astype(np.float64)
    if tag == F16:
        raw = x.astype(np.float16)
        return raw[0], raw[1], raw.astype(np.float64)
    return x[0], x[1], x.astype(np.float64)


def _fused(b, key_raw, val_raw, gpu, **kw):
    d = tl.device_batch(b, gpu)
    dist = torch.tensor([0, 0, b.n], dtype=torch.int32, device=gpu)
    out, pages = kernels.ragged_paged_attention_v3(d["query"], tl.to_torch(key_raw, b.kv_dtype, gpu), tl.to_torch(val_raw, b.kv_dtype, gpu),
                                                   d["kv_pages"], d["context_lens"], d["block_tables"].reshape(-1), d["query_start_loc"],
                                                   dist, num_kv_heads=b.Hkv, **kw)
    torch.cuda.synchronize()
    return tl.from_torch(out, b.q_dtype), pages


def test_unscaled_fp8_fused_write_is_a_bit_copy_of_the_cast_codes(gpu):
    b = tl.make_batch(311, [700, 65, 1500, 300], [1, 1, 2, 150], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=FP8, scaled=False)
    key_raw, val_raw, kv = _new_kv(np.random.default_rng(312), b.T, b.Hkv, b.D, FP8)
    want_codes = orc.page_scatter_ragged_ref(key_raw, val_raw, b.kv_raw, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
    got, pages = _fused(b, key_raw, val_raw, gpu)
    assert np.array_equal(pages.view(torch.uint8).cpu().numpy(), want_codes.astype(np.uint8)), "fp8 page write must copy the codes"
    want = tl.oracle_out(b, kv_val=orc.e4m3fn_bits_to_f32(want_codes.astype(np.uint8)).astype(np.float64))
    tl.assert_close(got, want, b, "unscaled fp8 fused")


def test_fp8_cache_through_the_v3_operation_is_cast_then_written(gpu, caplog):
    """kvdtype=float8_e4m3fn through the registry, as a model configured that way would run it: the view carries no
    scales, K/V are cast (round to nearest even, here far from overflow) and written, the attention reads the codes."""
    rng = np.random.default_rng(320)
    Hq, Hkv, D, pg, S, M = 32, 8, 128, 64, 3, 5
    P = S * M + 1
    cfg = RaggedPagesCacheConfig.create(torch.float8_e4m3fn, num_hidden_layers=1, num_kv_heads=Hkv, max_model_length=M * pg,
                                        kv_head_dim_size=D, page_size=pg, num_pages=P)
    assert cfg.get_shape_and_axes()[0] == (P, pg, 4, 4, 128)  # packing 4
    view = RaggedPagesCacheView.init(cfg, device=gpu)
    assert view.kv_scales is None
    bt = np.arange(1, P, dtype=np.int32).reshape(S, M)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    codes = np.zeros((P, pg, 2 * Hkv, D), np.uint8)
    ctx = np.zeros(S, np.int32)
    for q_lens in ([150, 70, 33], [1, 1, 40]):
        q_lens = np.array(q_lens, np.int32)
        ctx = (ctx + q_lens).astype(np.int32)
        qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
        T = int(qsl[-1])
        q_raw, k_raw, v_raw = (orc.f32_to_bf16_bits(rng.standard_normal((T, h, D), dtype=np.float32)) for h in (Hq, Hkv, Hkv))
        meta = RaggedPagesMetadata(pages_tables=torch.from_numpy(bt).to(gpu), context_lens=torch.from_numpy(ctx).to(gpu),
                                   query_start_loc=torch.from_numpy(qsl).to(gpu), num_seqs=torch.tensor([S], dtype=torch.int32, device=gpu),
                                   request_distribution=torch.from_numpy(orc.request_distribution_ref(q_lens, ctx)).to(gpu), page_size=pg)
        out = op(tl.to_torch(q_raw, BF16, gpu), tl.to_torch(k_raw, BF16, gpu), tl.to_torch(v_raw, BF16, gpu), view, meta)
        torch.cuda.synchronize()
        k8, v8 = orc.cast_e4m3fn_ref(orc.bf16_bits_to_f32(k_raw)), orc.cast_e4m3fn_ref(orc.bf16_bits_to_f32(v_raw))
        codes = orc.page_scatter_ragged_ref(k8, v8, codes, ctx, bt, qsl, [S]).astype(np.uint8)
        assert np.array_equal(view.kv_pages.view(torch.uint8).cpu().numpy().reshape(codes.shape), codes)
        want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(q_raw).astype(np.float64), orc.e4m3fn_bits_to_f32(codes).astype(np.float64),
                                              ctx, bt, qsl, [S])
        err = np.abs(tl.from_torch(out.attention_outputs, BF16) - want)
        assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN
    assert "lower-precision KV cache dtype" in caplog.text


# ---- padded head storage: D stored in rows of Dp = align(D, 128) ----------------------------------------------
@pytest.mark.parametrize("D,Dp,kv_dtype,q_dtype", [(96, 128, BF16, BF16), (80, 128, BF16, BF16), (192, 256, BF16, BF16),
                                                    (112, 128, FP8, BF16), (96, 128, F32, F32), (160, 256, BF16, F32)])
def test_padded_head_storage(gpu, D, Dp, kv_dtype, q_dtype):
    b = tl.make_batch(330 + D, [700, 65, 1500, 300, 33], [1, 1, 2, 150, 33], Hq=8, Hkv=2, D=D, page_size=32, q_dtype=q_dtype,
                      kv_dtype=kv_dtype, stored_dim=Dp, pad_rows=1, pad_tokens=2)
    kw = dict(sliding_window=900) if D == 80 else {}
    got = _check(b, f"padded heads D{D} in rows of {Dp}", **kw)
    assert got.shape[-1] == D
    # every row tile of the prefill kernel split over key chunks, and every decode row merged from partial slots
    if q_dtype == BF16:
        prev = (_lib.set_tunable("prefill_chunks", 4), _lib.set_tunable("decode_wgs", 7))
        try:
            b2 = tl.make_batch(331 + D, [9000, 20000], [1, 200], Hq=8, Hkv=2, D=D, page_size=32, kv_dtype=kv_dtype, stored_dim=Dp)
            _check(b2, f"padded heads D{D}, rows in pieces")
        finally:
            _lib.set_tunable("prefill_chunks", prev[0])
            _lib.set_tunable("decode_wgs", prev[1])


@pytest.mark.parametrize("kv_dtype", [BF16, F32])
def test_padded_head_fused_write_places_rows_and_zeroes_the_padding(gpu, kv_dtype):
    D, Dp = 96, 128
    b = tl.make_batch(340, [700, 65, 1500, 300], [1, 1, 2, 150], Hq=8, Hkv=2, D=D, page_size=32, q_dtype=kv_dtype, kv_dtype=kv_dtype,
                      stored_dim=Dp)
    b.kv_dev = tl.device_pool(b)
    b.kv_dev[..., D:] = 7 if kv_dtype == F32 else 0x4000  # stale, finite padding: the write must zero it where it writes
    key_raw, val_raw, _ = _new_kv(np.random.default_rng(341), b.T, b.Hkv, D, kv_dtype)
    want_pages = orc.page_scatter_ragged_ref(key_raw, val_raw, b.kv_raw, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
    got, pages = _fused(b, key_raw, val_raw, gpu)
    pages = pages.view(torch.int16).cpu().numpy().view(np.uint16) if kv_dtype == BF16 else pages.cpu().numpy()
    assert np.array_equal(pages[..., :D], want_pages.astype(pages.dtype)), "rows of the padded pool"
    written = np.zeros(pages.shape[:2], bool)  # (page, slot) pairs the call wrote
    for i in range(b.n):
        q_len = int(b.q_lens[i])
        for pos in range(int(b.context_lens[i]) - q_len, int(b.context_lens[i])):
            written[b.block_tables[i, pos // b.page_size], pos % b.page_size] = True
    assert not pages[written][..., D:].any(), "padding of written rows must be zero"
    assert np.array_equal(pages[~written][..., D:], b.kv_dev[~written][..., D:]), "rows not written keep their bytes"
    vals = orc.bf16_bits_to_f32(want_pages.astype(np.uint16)).astype(np.float64) if kv_dtype == BF16 else want_pages.astype(np.float64)
    tl.assert_close(got, tl.oracle_out(b, kv_val=vals), b, "padded heads, fused")
    # the stand-alone ragged write does the same
    d = tl.device_batch(b, gpu)
    kernels.page_scatter_ragged(tl.to_torch(key_raw, kv_dtype, gpu), tl.to_torch(val_raw, kv_dtype, gpu), d["kv_pages"], d["context_lens"],
                                d["block_tables"], d["query_start_loc"], d["num_seqs"])
    torch.cuda.synchronize()
    alone = d["kv_pages"].view(torch.int16).cpu().numpy().view(np.uint16) if kv_dtype == BF16 else d["kv_pages"].cpu().numpy()
    assert np.array_equal(alone, pages)


def test_padded_heads_through_the_v3_operation(gpu):
    """head_dim 96 through the registry: the config stores rows of 128 (v3 shape [P, pg, groups, packing, 128])."""
    rng = np.random.default_rng(350)
    Hq, Hkv, D, pg, S, M = 8, 2, 96, 32, 3, 8
    P = S * M + 1
    cfg = RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=Hkv, max_model_length=M * pg,
                                        kv_head_dim_size=D, page_size=pg, num_pages=P)
    assert cfg.get_shape_and_axes()[0] == (P, pg, 2, 2, 128) and cfg.combined_heads_per_token == 4
    view = RaggedPagesCacheView.init(cfg, device=gpu)
    bt = np.arange(1, P, dtype=np.int32).reshape(S, M)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    vals = np.zeros((P, pg, 2 * Hkv, D), np.uint16)
    ctx = np.zeros(S, np.int32)
    for q_lens in ([150, 70, 33], [1, 1, 40]):
        q_lens = np.array(q_lens, np.int32)
        ctx = (ctx + q_lens).astype(np.int32)
        qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
        T = int(qsl[-1])
        q_raw, k_raw, v_raw = (orc.f32_to_bf16_bits(rng.standard_normal((T, h, D), dtype=np.float32)) for h in (Hq, Hkv, Hkv))
        meta = RaggedPagesMetadata(pages_tables=torch.from_numpy(bt).to(gpu), context_lens=torch.from_numpy(ctx).to(gpu),
                                   query_start_loc=torch.from_numpy(qsl).to(gpu), num_seqs=torch.tensor([S], dtype=torch.int32, device=gpu),
                                   request_distribution=torch.from_numpy(orc.request_distribution_ref(q_lens, ctx)).to(gpu), page_size=pg)
        out = op(tl.to_torch(q_raw, BF16, gpu)[None], tl.to_torch(k_raw, BF16, gpu)[None], tl.to_torch(v_raw, BF16, gpu)[None], view, meta)
        torch.cuda.synchronize()
        assert tuple(out.attention_outputs.shape) == (1, T, Hq, D)
        vals = orc.page_scatter_ragged_ref(k_raw, v_raw, vals, ctx, bt, qsl, [S]).astype(np.uint16)
        stored = view.kv_pages.view(torch.int16).cpu().numpy().view(np.uint16).reshape(P, pg, 2 * Hkv, 128)
        assert np.array_equal(stored[..., :D], vals) and not stored[..., D:].any()
        want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(q_raw).astype(np.float64), orc.bf16_bits_to_f32(vals).astype(np.float64),
                                              ctx, bt, qsl, [S])
        err = np.abs(tl.from_torch(out.attention_outputs[0], BF16) - want)
        assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN


# ---- float16 queries and pages (the fp32 kernel serves them) -----------------------------------------------------
@pytest.mark.parametrize("q_dtype,kv_dtype", [(F16, F16), (F16, F32), (F32, F16), (BF16, F16)])
def test_float16_queries_and_pages(gpu, q_dtype, kv_dtype):
    b = tl.make_batch(360, [17, 64, 130, 255, 700], [1, 1, 8, 33, 2], Hq=8, Hkv=2, D=64, page_size=16, q_dtype=q_dtype,
                      kv_dtype=kv_dtype, pad_rows=1, pad_tokens=2)
    got = _check(b, f"q {q_dtype} kv {kv_dtype}", sliding_window=300, logits_soft_cap=20.0)
    assert np.all(got[int(b.query_start_loc[b.n]):] == 0.0), "padded token rows must be written as zeros"
    if q_dtype == kv_dtype == F16:  # the fused write copies float16 rows bit for bit
        key_raw, val_raw, _ = _new_kv(np.random.default_rng(361), b.T, b.Hkv, b.D, F16)
        want_pages = orc.page_scatter_ragged_ref(key_raw, val_raw, b.kv_raw, b.context_lens, b.block_tables, b.query_start_loc, b.num_seqs)
        got, pages = _fused(b, key_raw, val_raw, gpu)
        assert np.array_equal(pages.cpu().numpy(), want_pages.astype(np.float16))
        tl.assert_close(got, tl.oracle_out(b, kv_val=want_pages.astype(np.float64)), b, "float16 fused")


# ---- query rows before position 0 (q_len > context_len) see no key: zeros from every kernel -------------------------
@pytest.mark.parametrize("kv_dtype,dma", [(BF16, 1), (BF16, 0), (FP8, 1), (F32, 1)])
def test_rows_before_position_zero_are_zeros_on_every_kernel(gpu, kv_dtype, dma):
    """A 400-token chunk over a 100-token context: the first 300 query tokens sit at negative positions.  Their
    row tiles hold no key at all (the MFMA prefill kernels' keyless-tile path) or only some rows with keys."""
    q_dtype = F32 if kv_dtype == F32 else BF16
    b = tl.make_batch(370, [100, 700, 5], [400, 1, 9], Hq=8, Hkv=2, D=128, page_size=32, q_dtype=q_dtype, kv_dtype=kv_dtype)
    d = tl.device_batch(b, gpu)
    prev = _lib.set_tunable("prefill_dma", dma)
    try:
        out = torch.full_like(d["query"], float("nan"))  # rows nobody writes would stay NaN
        kernels.ragged_paged_attention(d["query"], d["kv_pages"], d["context_lens"], d["block_tables"], d["query_start_loc"], d["num_seqs"],
                                       kv_scales=d["kv_scales"], num_kv_heads=b.Hkv, out=out)
        torch.cuda.synchronize()
    finally:
        _lib.set_tunable("prefill_dma", prev)
    got = tl.from_torch(out, q_dtype)
    want = tl.oracle_out(b)
    assert not want[:300].any() and not want[401:405].any()
    tl.assert_close(got, want, b, "rows before position 0")
    assert not got[:300].any() and not got[401:405].any()


# ---- 8-bit pages on the LDS-direct prefill pipeline ------------------------------------------------------------------
@pytest.mark.parametrize("kv_dtype", [FP8, tl.INT8])
@pytest.mark.parametrize("D,page_size,Hq,Hkv", [(128, 64, 32, 8), (256, 32, 8, 4), (128, 128, 40, 8)])
def test_8bit_prefill_on_the_lds_direct_pipeline(gpu, kv_dtype, D, page_size, Hq, Hkv):
    """Chunked prefill over scaled 8-bit pages: the kernel that loads codes straight into LDS and widens them there,
    against the oracle and against the register-staged kernel; with a window whose left edge falls inside a tile, a
    soft cap, a row tile split over key chunks, and NaN codes in the slots past the context."""
    b = tl.make_batch(400 + D + page_size, [3000, 700, 9300, 40], [300, 1, 520, 40], Hq=Hq, Hkv=Hkv, D=D, page_size=page_size,
                      kv_dtype=kv_dtype, pad_rows=1, pad_tokens=3)
    if kv_dtype == FP8:  # slots past each context hold NaN codes: nobody may read them as data
        for i, c in enumerate(b.context_lens[:b.n]):
            if c % page_size:
                b.kv_raw[b.block_tables[i, c // page_size], c % page_size:] = 0x7F
    for kw in ({}, dict(sliding_window=777, logits_soft_cap=30.0)):
        # (scales up to 2 on N(0,1) codes: rows that see a handful of keys return values beyond 4, where a bf16 result
        # cannot keep 2e-2)
        got = _check(b, f"8-bit prefill kv{kv_dtype} D{D} pg{page_size} {sorted(kw)}", above_4=True, **kw)
        prev = _lib.set_tunable("prefill_dma", 0)
        try:
            staged = tl.run_gpu_attention(b, **kw)
        finally:
            _lib.set_tunable("prefill_dma", prev)
        tl.assert_close(staged, tl.oracle_out(b, **kw), b, "register-staged kernel")
        # (the two kernels round V differently -- bf16(code x scale) here, code x scale in float32 there -- so they
        # agree with each other only as closely as each agrees with the oracle)
        assert np.abs(got - staged)[tl.valid_rows(b)].max() <= 2 * tl.TOL_BF16_MAX
    prev = _lib.set_tunable("prefill_chunks", 8)
    try:
        b2 = tl.make_batch(401 + D, [20000], [200], Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype)
        _check(b2, "8-bit prefill, row tiles split over key chunks", above_4=True)
    finally:
        _lib.set_tunable("prefill_chunks", prev)
