"""GPU tests of the quantising page write (scaled fp8 / int8 pages): bit-exact against the oracle's rule, over
several serving steps, and the attention that follows it."""

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd import kernels
from easydel_amd.caching import RaggedPagesCacheConfig, RaggedPagesCacheView, RaggedPagesMetadata
from easydel_amd.operations import OperationMetadata, OperationRegistry
from rpa_testlib import BF16, F32, FP8, INT8, orc

pytestmark = pytest.mark.gpu

TORCH_KV = {FP8: torch.float8_e4m3fn, INT8: torch.int8}


def _tables(rng, S, M, P):
    perm = rng.permutation(np.arange(1, P)).astype(np.int32)
    return perm[:S * M].reshape(S, M)


def _gpu_write(key, value, src_tag, codes, scales, ctx, bt, qsl, n_live, kv_dtype, dev):
    k = tl.to_torch(key, src_tag, dev)
    v = tl.to_torch(value, src_tag, dev)
    pages = torch.from_numpy(codes.copy()).to(dev).view(TORCH_KV[kv_dtype])
    sc = torch.from_numpy(scales.copy()).to(dev)
    kernels.page_scatter_ragged_quantised(k, v, pages, sc, torch.from_numpy(ctx).to(dev), torch.from_numpy(bt).to(dev),
                                          torch.from_numpy(qsl).to(dev), torch.tensor([n_live], dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    return pages.view(torch.uint8).cpu().numpy(), sc.cpu().numpy()


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
@pytest.mark.parametrize("src_tag,D,pg,Hkv", [(BF16, 128, 64, 8), (F32, 64, 16, 2), (BF16, 256, 32, 4)])
def test_quantising_write_is_bit_exact_over_serving_steps(gpu, kv_dtype, src_tag, D, pg, Hkv):
    # a prefill step, a chunked-prefill step and decode steps on the same pages: scales grow, old tokens are re-coded
    rng = np.random.default_rng(90 + D + kv_dtype)
    S, M, P = 5, 6, 40
    bt = _tables(rng, S, M, P)
    codes = rng.integers(0, 255, size=(P, pg, 2 * Hkv, D), dtype=np.uint8)  # stale contents of recycled pages
    scales = rng.uniform(0.5, 4.0, size=(P, 2 * Hkv)).astype(np.float32)     # stale scales: must be ignored on a fresh page
    ctx = np.zeros(S, np.int32)
    steps = [[pg + 5, 3, 1, 2 * pg, 0], [1, pg - 3, 1, 7, 9], [1, 1, 1, 1, 1], [1, 1, 0, 1, 1], [3, 1, 1, 1, pg]]
    for step, q_lens in enumerate(steps):
        q_lens = np.array(q_lens, np.int32)
        ctx = (ctx + q_lens).astype(np.int32)
        qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
        T = int(qsl[-1])
        gain = 1.0 + 0.6 * step  # later steps carry larger values, so stored scales must grow
        k = (rng.standard_normal((T, Hkv, D)) * gain).astype(np.float32)
        v = (rng.standard_normal((T, Hkv, D)) * gain).astype(np.float32)
        if src_tag == BF16:
            k_raw, v_raw = orc.f32_to_bf16_bits(k), orc.f32_to_bf16_bits(v)
            k, v = orc.bf16_bits_to_f32(k_raw), orc.bf16_bits_to_f32(v_raw)
        else:
            k_raw, v_raw = k, v
        ctx_step = np.where(q_lens > 0, ctx, 0).astype(np.int32)
        want_codes, want_scales = orc.page_scatter_ragged_quantised_ref(k, v, codes, scales, ctx_step, bt, qsl, [S], kv_dtype=kv_dtype)
        got_codes, got_scales = _gpu_write(k_raw, v_raw, src_tag, codes, scales, ctx_step, bt, qsl, S, kv_dtype, gpu)
        assert np.array_equal(got_scales, want_scales), f"step {step}: scales differ"
        assert np.array_equal(got_codes, want_codes), f"step {step}: {np.count_nonzero(got_codes != want_codes)} codes differ"
        codes, scales = got_codes, got_scales
    # what the pages now hold is close to what was written last: half a code step at the page's scale
    last = ctx[0] - 1
    page, off = bt[0, last // pg], last % pg
    deq = orc.decode_codes(codes[page, off], kv_dtype) * scales[page][:, None]
    truth = np.stack([k[qsl[1] - 1], v[qsl[1] - 1]], axis=1).reshape(2 * Hkv, D)
    step_size = scales[page][:, None] * (32.0 if kv_dtype == FP8 else 1.0)  # largest code spacing: 32 at |code| >= 256
    assert (np.abs(deq - truth) <= 0.5 * step_size + 1e-6).all()


def test_quantising_write_skips_padding_and_other_pages(gpu):
    rng = np.random.default_rng(7)
    S, M, P, pg, Hkv, D = 4, 3, 16, 16, 2, 64
    bt = _tables(rng, S, M, P)
    codes = rng.integers(0, 255, size=(P, pg, 2 * Hkv, D), dtype=np.uint8)
    scales = rng.uniform(0.5, 4.0, size=(P, 2 * Hkv)).astype(np.float32)
    ctx = np.array([20, 7, 0, 0], np.int32)
    qsl = np.array([0, 2, 9, 9, 9], np.int32)  # 2 live rows, then padded rows; 3 padded tokens follow
    k = rng.standard_normal((12, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((12, Hkv, D)).astype(np.float32)
    want = orc.page_scatter_ragged_quantised_ref(k, v, codes, scales, ctx, bt, qsl, [2], kv_dtype=INT8)
    got = _gpu_write(k, v, F32, codes, scales, ctx, bt, qsl, 2, INT8, gpu)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    touched = {int(bt[0, 1]), int(bt[1, 0])}
    for page in range(P):
        if page not in touched:
            assert np.array_equal(got[0][page], codes[page]) and np.array_equal(got[1][page], scales[page])


@pytest.mark.parametrize("kv_dtype", [FP8, INT8])
def test_fused_quantised_v3_operation(gpu, kv_dtype):
    # registry -> v3 operation on a view with scales: writes the step's K/V quantised, then attends; twice
    rng = np.random.default_rng(11)
    Hq, Hkv, D, pg, S, M = 32, 8, 128, 64, 4, 6
    P = S * M + 1
    cfg = RaggedPagesCacheConfig.create(TORCH_KV[kv_dtype], num_hidden_layers=1, num_kv_heads=Hkv, max_model_length=M * pg,
                                        kv_head_dim_size=D, page_size=pg, num_pages=P)
    view = RaggedPagesCacheView.init(cfg, device=gpu, scaled=True)
    bt = _tables(rng, S, M, P)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    codes = np.zeros((P, pg, 2 * Hkv, D), np.uint8)
    scales = np.ones((P, 2 * Hkv), np.float32)
    ctx = np.zeros(S, np.int32)
    for q_lens in ([150, 70, 1, 33], [1, 1, 1, 40]):
        q_lens = np.array(q_lens, np.int32)
        ctx = (ctx + q_lens).astype(np.int32)
        qsl = np.concatenate([[0], np.cumsum(q_lens)]).astype(np.int32)
        T = int(qsl[-1])
        q_raw, k_raw, v_raw = (orc.f32_to_bf16_bits(rng.standard_normal((T, h, D), dtype=np.float32)) for h in (Hq, Hkv, Hkv))
        dist = orc.request_distribution_ref(q_lens, ctx)
        meta = RaggedPagesMetadata(pages_tables=torch.from_numpy(bt).to(gpu), context_lens=torch.from_numpy(ctx).to(gpu),
                                   query_start_loc=torch.from_numpy(qsl).to(gpu), num_seqs=torch.tensor([S], dtype=torch.int32, device=gpu),
                                   request_distribution=torch.from_numpy(dist).to(gpu), page_size=pg)
        out = op(tl.to_torch(q_raw, BF16, gpu), tl.to_torch(k_raw, BF16, gpu), tl.to_torch(v_raw, BF16, gpu), view, meta)
        torch.cuda.synchronize()
        codes, scales = orc.page_scatter_ragged_quantised_ref(orc.bf16_bits_to_f32(k_raw), orc.bf16_bits_to_f32(v_raw), codes, scales,
                                                              ctx, bt, qsl, [S], kv_dtype=kv_dtype)
        assert np.array_equal(view.kv_pages.view(torch.uint8).cpu().numpy().reshape(codes.shape), codes)
        assert np.array_equal(view.kv_scales.cpu().numpy(), scales)
        kv_val = orc.decode_codes(codes, kv_dtype).astype(np.float64) * scales[:, None, :, None]
        want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(q_raw).astype(np.float64), kv_val, ctx, bt, qsl, [S])
        got = tl.from_torch(out.attention_outputs, BF16)
        err = np.abs(got - want)
        assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN
        # and the dequantised attention stays close to attention over the unquantised history of this step's keys
        assert out.cache_view is view
