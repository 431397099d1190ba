"""GPU parity of the unified-attention layout (separate K and V pools) through the C ABI and the operation."""

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd.caching import (RaggedPagesMetadata, UnifiedAttentionCacheConfig, UnifiedAttentionCacheView,
                                 compute_ragged_batch_fields)
from easydel_amd.operations import AttentionOutput, OperationMetadata, OperationRegistry
from rpa_testlib import BF16, F32, FP8, INT8, orc

pytestmark = pytest.mark.gpu


def _check(b, what, **kw):
    got = tl.run_gpu_unified_attention(b, **kw)
    want = tl.oracle_out(b, **kw)
    mx, mean = tl.assert_close(got, want, b, what)
    print(f"{what}: max-abs {mx:.3e} mean-abs {mean:.3e}", flush=True)
    return got


@pytest.mark.parametrize("D,page_size,Hq,Hkv,kv_dtype", [
    (128, 64, 32, 8, BF16), (64, 16, 8, 2, BF16), (256, 128, 16, 8, BF16), (128, 32, 8, 8, BF16), (64, 64, 32, 1, BF16),
    (128, 64, 40, 8, FP8), (128, 32, 8, 8, INT8), (64, 16, 8, 2, F32)])
def test_unified_mixed_batch(gpu, D, page_size, Hq, Hkv, kv_dtype):
    # decode rows, multi-token small rows, chunked and full prefill in one batch, padded rows and tokens
    ctx = [300, 1000, 129, 47, 2100, 700, 5, 1]
    q_lens = [300, 200, 129, 33, 17, 1, 2, 1]
    b = tl.make_batch(80 + D, ctx, q_lens, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, kv_dtype=kv_dtype,
                      q_dtype=F32 if kv_dtype == F32 else BF16, pad_rows=2, pad_tokens=5)
    got = _check(b, f"unified D{D} pg{page_size} {Hq}/{Hkv} kv{kv_dtype}")
    # the kernels are the same and so is the order of their arithmetic: only addresses differ between the layouts
    assert np.array_equal(got[tl.valid_rows(b)], tl.run_gpu_attention(b)[tl.valid_rows(b)])


def test_unified_c1_fp32(gpu):
    b = tl.make_batch(0, [17, 64, 130, 255], [1, 1, 8, 33], Hq=8, Hkv=2, D=64, page_size=16, num_pages=128,
                      q_dtype=F32, kv_dtype=F32)
    _check(b, "unified C1 fp32", softmax_scale=1.0 / 8.0)


@pytest.mark.parametrize("window,cap", [(100, None), (None, 30.0), (513, 50.0)])
def test_unified_window_and_soft_cap(gpu, window, cap):
    ctx = [600, 1500, 640, 64, 900, 77]
    q_lens = [600, 300, 40, 64, 1, 1]
    b = tl.make_batch(81, ctx, q_lens, Hq=16, Hkv=4, D=128, page_size=64, max_pages=24)
    _check(b, f"unified window {window} cap {cap}", sliding_window=window, logits_soft_cap=cap)


def test_unified_without_live_row_count(gpu):
    # the reference's kernel takes no row count: padded rows are recognised by their empty query span
    ctx = [900, 33, 1, 260]
    q_lens = [1, 33, 1, 130]
    b = tl.make_batch(82, ctx, q_lens, Hq=32, Hkv=8, D=128, page_size=64, pad_rows=5)
    with_count = _check(b, "unified, row count given")
    without = tl.run_gpu_unified_attention(b, pass_num_seqs=False)
    tl.assert_close(without, tl.oracle_out(b), b, "unified, no row count")
    assert np.array_equal(with_count[tl.valid_rows(b)], without[tl.valid_rows(b)])


def test_unified_operation_with_cache_update(gpu):
    # registry -> UnifiedAttn, pools written by the view's concatenate_to_cache with the v2 slot mapping
    rng = np.random.default_rng(5)
    Hq, Hkv, D, pg = 32, 8, 128, 64
    scheduled, computed = [1, 1, 40, 130], [300, 63, 0, 100]
    max_reqs, max_pages = 6, 8
    n_pages = max_reqs * max_pages + 1
    table = np.zeros((max_reqs, max_pages), dtype=np.int32)
    perm = rng.permutation(np.arange(1, n_pages))
    k = 0
    for r in range(len(scheduled)):
        need = -(-(computed[r] + scheduled[r]) // pg)
        table[r, :need] = perm[k:k + need]
        k += need
    cfg = UnifiedAttentionCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=Hkv,
                                             max_model_length=max_pages * pg, head_dim=D, page_size=pg, num_pages=n_pages)
    sched_full = np.zeros(max_reqs, np.int32); sched_full[:len(scheduled)] = scheduled
    comp_full = np.zeros(max_reqs, np.int32); comp_full[:len(computed)] = computed
    fields = compute_ragged_batch_fields(scheduled_full=sched_full, active_mask_full=sched_full > 0, num_computed_tokens=comp_full,
                                         page_table=table, version="v2", max_num_reqs=max_reqs, page_size=pg)
    view = UnifiedAttentionCacheView.init(cfg, device=gpu)
    assert tuple(view.key_cache.shape) == tuple(view.value_cache.shape) == (n_pages, pg, Hkv, D)
    k_pool = orc.f32_to_bf16_bits(rng.standard_normal(view.key_cache.shape, dtype=np.float32))
    v_pool = orc.f32_to_bf16_bits(rng.standard_normal(view.value_cache.shape, dtype=np.float32))
    view.key_cache.copy_(tl.to_torch(k_pool, BF16, gpu))
    view.value_cache.copy_(tl.to_torch(v_pool, BF16, gpu))
    T = int(sum(scheduled))
    q_raw, k_raw, v_raw = (orc.f32_to_bf16_bits(rng.standard_normal((T, h, D), dtype=np.float32)) for h in (Hq, Hkv, Hkv))
    meta = RaggedPagesMetadata.from_numpy(fields, version="v2", page_size=pg, device=gpu)
    key, value = tl.to_torch(k_raw, BF16, gpu), tl.to_torch(v_raw, BF16, gpu)
    assert view.concatenate_to_cache(key[None], value[None], meta) is view
    op = OperationRegistry.create("unified_attention", OperationMetadata())
    out = op(tl.to_torch(q_raw, BF16, gpu)[None], view, meta, sliding_window=128, causal=True, deterministic=True)
    torch.cuda.synchronize()
    assert isinstance(out, AttentionOutput) and out.cache_view is view and out.attention_weights is None
    assert tuple(out.attention_outputs.shape) == (1, T, Hq, D)
    # bit-exact pools after the update, each checked against the slice-scatter oracle on its own rows
    k_after = orc.kv_cache_update_ref(k_raw, fields["slot_mapping"], k_pool.reshape(-1, Hkv, D),
                                      fields["num_kv_update_slices"], page_size=pg).reshape(k_pool.shape)
    v_after = orc.kv_cache_update_ref(v_raw, fields["slot_mapping"], v_pool.reshape(-1, Hkv, D),
                                      fields["num_kv_update_slices"], page_size=pg).reshape(v_pool.shape)
    assert np.array_equal(view.key_cache.view(torch.int16).cpu().numpy().view(np.uint16), k_after)
    assert np.array_equal(view.value_cache.view(torch.int16).cpu().numpy().view(np.uint16), v_after)
    pages = np.stack([k_after, v_after], axis=3).reshape(n_pages, pg, 2 * Hkv, D)  # K at even, V at odd combined heads
    want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(q_raw).astype(np.float64), orc.bf16_bits_to_f32(pages).astype(np.float64),
                                          fields["context_lens"], fields["pages_tables"], fields["query_start_loc"],
                                          np.array([max_reqs], np.int32), sliding_window=128)
    assert np.abs(tl.from_torch(out.attention_outputs[0], BF16) - want).max() <= tl.TOL_BF16_MAX


def test_unified_operation_rejects_what_the_kernels_do_not_cover(gpu):
    op = OperationRegistry.create("unified_attention", OperationMetadata())
    q = torch.zeros((2, 8, 64), device=gpu, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        op(q, None, None)
    cfg = UnifiedAttentionCacheConfig.create(torch.bfloat16, 1, 2, 64, 64, page_size=16, num_pages=4)
    view = UnifiedAttentionCacheView.init(cfg, device=gpu)
    meta = RaggedPagesMetadata.create_empty(2, 2, 4, page_size=16, version="v2", device=gpu)
    with pytest.raises(NotImplementedError, match="one sink logit per query head"):
        op(q, view, meta, softmax_aux=torch.zeros(2, device=gpu))  # 8 query heads
    with pytest.raises(NotImplementedError):
        op(q, view, meta, causal=False)
