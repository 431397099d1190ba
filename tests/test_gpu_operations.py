"""GPU tests of the operation-level drop-in: registry -> RaggedPageAttnV2/V3 -> C ABI, against the oracle."""

import logging

import numpy as np
import pytest
import torch

import rpa_testlib as tl
from easydel_amd.caching import RaggedPagesCacheConfig, RaggedPagesCacheView, RaggedPagesMetadata, compute_ragged_batch_fields
from easydel_amd.operations import AttentionOutput, OperationMetadata, OperationRegistry
from rpa_testlib import BF16, F32, orc

pytestmark = pytest.mark.gpu


def _scenario(rng, *, Hq, Hkv, D, page_size, dtype, version, scheduled, computed, max_reqs, max_pages):
    """Scheduler-shaped inputs: per-request scheduled / computed token counts and a page table."""
    n_pages = max_reqs * max_pages + 1
    table = np.zeros((max_reqs, max_pages), dtype=np.int32)
    perm = rng.permutation(np.arange(1, n_pages))
    k = 0
    for r in range(len(scheduled)):
        need = -(-(computed[r] + scheduled[r]) // page_size)
        table[r, :need] = perm[k:k + need]
        k += need
    cfg = RaggedPagesCacheConfig.create(dtype, num_hidden_layers=1, num_kv_heads=Hkv, max_model_length=max_pages * page_size,
                                        kv_head_dim_size=D, page_size=page_size, num_pages=n_pages, version=version)
    sched_full = np.zeros(max_reqs, np.int32); sched_full[:len(scheduled)] = scheduled
    comp_full = np.zeros(max_reqs, np.int32); comp_full[:len(computed)] = computed
    fields = compute_ragged_batch_fields(scheduled_full=sched_full, active_mask_full=sched_full > 0, num_computed_tokens=comp_full,
                                         page_table=table, version=version, max_num_reqs=max_reqs, page_size=page_size)
    return cfg, fields


@pytest.mark.parametrize("np_dtype,torch_dtype,tag,D,page_size,Hq,Hkv", [
    (np.float32, torch.float32, F32, 64, 16, 8, 2), (None, torch.bfloat16, BF16, 128, 64, 32, 8), (None, torch.bfloat16, BF16, 256, 128, 16, 8)])
def test_v3_operation_end_to_end(gpu, np_dtype, torch_dtype, tag, D, page_size, Hq, Hkv):
    rng = np.random.default_rng(1)
    scheduled, computed = [1, 1, 8, 33, 70], [16, 63, 122, 222, 0]
    cfg, fields = _scenario(rng, Hq=Hq, Hkv=Hkv, D=D, page_size=page_size, dtype=torch_dtype, version="v3",
                            scheduled=scheduled, computed=computed, max_reqs=8, max_pages=24)
    view = RaggedPagesCacheView.init(cfg, layer_index=0, device=gpu)
    assert view.kv_pages.ndim == 5
    shape4 = (cfg.num_pages, page_size, 2 * Hkv, D)
    pool = rng.standard_normal(shape4, dtype=np.float32)
    T = int(sum(scheduled))
    q = rng.standard_normal((1, T, Hq, D), dtype=np.float32)
    k = rng.standard_normal((1, T, Hkv, D), dtype=np.float32)
    v = rng.standard_normal((1, T, Hkv, D), dtype=np.float32)
    if tag == BF16:
        pool_raw, q_raw, k_raw, v_raw = (orc.f32_to_bf16_bits(a) for a in (pool, q, k, v))
        dec = lambda a: orc.bf16_bits_to_f32(a).astype(np.float64)  # noqa: E731
    else:
        pool_raw, q_raw, k_raw, v_raw = pool, q, k, v
        dec = lambda a: a.astype(np.float64)  # noqa: E731
    view.kv_pages.copy_(tl.to_torch(pool_raw, tag, gpu).view(view.kv_pages.shape))
    meta = RaggedPagesMetadata.from_numpy(fields, version="v3", page_size=page_size, device=gpu)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    out = op(tl.to_torch(q_raw, tag, gpu), tl.to_torch(k_raw, tag, gpu), tl.to_torch(v_raw, tag, gpu), view, meta,
             softmax_scale=None, sliding_window=None, logits_soft_cap=None, causal=True, deterministic=True, bias=None)
    torch.cuda.synchronize()
    assert isinstance(out, AttentionOutput) and out.attention_weights is None and out.cache_view is view
    assert tuple(out.attention_outputs.shape) == (1, T, Hq, D) and out.attention_outputs.dtype == torch_dtype
    pages_after = orc.page_scatter_ragged_ref(k_raw[0], v_raw[0], pool_raw, fields["context_lens"], fields["pages_tables"],
                                              fields["query_start_loc"], fields["num_seqs"])
    got_pages = view.kv_pages.view(torch.uint8).cpu().numpy()
    assert np.array_equal(got_pages, pages_after.view(np.uint8).reshape(got_pages.shape)), "page scatter must be bit-exact"
    want = orc.ragged_paged_attention_ref(dec(q_raw[0]), dec(pages_after), fields["context_lens"], fields["pages_tables"],
                                          fields["query_start_loc"], fields["num_seqs"])
    err = np.abs(tl.from_torch(out.attention_outputs[0], tag) - want)
    assert err.max() <= (tl.TOL_F32_MAX if tag == F32 else tl.TOL_BF16_MAX)


def test_v2_operation_with_cache_update(gpu):
    rng = np.random.default_rng(2)
    Hq, Hkv, D, pg = 32, 8, 128, 64
    scheduled, computed = [1, 1, 40, 130], [300, 63, 0, 100]
    cfg, fields = _scenario(rng, Hq=Hq, Hkv=Hkv, D=D, page_size=pg, dtype=torch.bfloat16, version="v2",
                            scheduled=scheduled, computed=computed, max_reqs=6, max_pages=8)
    view = RaggedPagesCacheView.init(cfg, device=gpu)
    assert tuple(view.kv_pages.shape) == (cfg.num_pages, pg, 2 * Hkv, D)
    pool_raw = orc.f32_to_bf16_bits(rng.standard_normal(view.kv_pages.shape, dtype=np.float32))
    view.kv_pages.copy_(tl.to_torch(pool_raw, BF16, gpu))
    T = int(sum(scheduled))
    q_raw, k_raw, v_raw = (orc.f32_to_bf16_bits(rng.standard_normal((T, h, D), dtype=np.float32)) for h in (Hq, Hkv, Hkv))
    meta = RaggedPagesMetadata.from_numpy(fields, version="v2", page_size=pg, device=gpu)
    key, value = tl.to_torch(k_raw, BF16, gpu), tl.to_torch(v_raw, BF16, gpu)
    assert view.concatenate_to_cache(key[None], value[None], meta) is view
    op = OperationRegistry.create("ragged_page_attention_v2", OperationMetadata())
    out = op(tl.to_torch(q_raw, BF16, gpu), key, value, view, meta, sliding_window=128)
    torch.cuda.synchronize()
    new_kv = np.stack([k_raw, v_raw], axis=2).reshape(T, 2 * Hkv, D)
    pages_after = orc.kv_cache_update_ref(new_kv, fields["slot_mapping"], pool_raw.reshape(-1, 2 * Hkv, D),
                                          fields["num_kv_update_slices"], page_size=pg).reshape(pool_raw.shape)
    assert np.array_equal(view.kv_pages.view(torch.int16).cpu().numpy().view(np.uint16), pages_after)
    want = orc.ragged_paged_attention_ref(orc.bf16_bits_to_f32(q_raw).astype(np.float64), orc.bf16_bits_to_f32(pages_after).astype(np.float64),
                                          fields["context_lens"], fields["pages_tables"], fields["query_start_loc"], fields["num_seqs"],
                                          sliding_window=128)
    assert tuple(out.attention_outputs.shape) == (T, Hq, D) and out.cache_view is None
    assert np.abs(tl.from_torch(out.attention_outputs, BF16) - want).max() <= tl.TOL_BF16_MAX


def test_v3_casts_key_value_to_cache_dtype_with_warning(gpu, caplog):
    rng = np.random.default_rng(3)
    cfg, fields = _scenario(rng, Hq=8, Hkv=2, D=64, page_size=16, dtype=torch.bfloat16, version="v3",
                            scheduled=[3, 1], computed=[5, 40], max_reqs=2, max_pages=4)
    view = RaggedPagesCacheView.init(cfg, device=gpu)
    meta = RaggedPagesMetadata.from_numpy(fields, version="v3", page_size=16, device=gpu)
    q = torch.randn((4, 8, 64), device=gpu, dtype=torch.bfloat16)
    k32, v32 = torch.randn((4, 2, 64), device=gpu), torch.randn((4, 2, 64), device=gpu)
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    with caplog.at_level(logging.WARNING):
        op(q, k32, v32, view, meta)
    torch.cuda.synchronize()
    assert "lower-precision KV cache dtype" in caplog.text
    page, slot = int(fields["pages_tables"][1, 40 // 16]), 40 % 16
    stored = view.kv_pages.view(cfg.num_pages, 16, 4, 64)[page, slot]
    assert torch.equal(stored[0], k32[3, 0].to(torch.bfloat16)) and torch.equal(stored[1], v32[3, 0].to(torch.bfloat16))


def test_quantised_view_is_read_through_scales(gpu):
    b = tl.make_batch(60, [700, 65, 1500], [1, 1, 40], Hq=32, Hkv=8, D=128, page_size=64, kv_dtype=tl.FP8)
    d = tl.device_batch(b, gpu)
    cfg = RaggedPagesCacheConfig.create(torch.float8_e4m3fn, num_hidden_layers=1, num_kv_heads=8, max_model_length=b.M * 64,
                                        kv_head_dim_size=128, page_size=64, num_pages=b.P)
    assert RaggedPagesCacheView.init(cfg, device=gpu).kv_scales is None  # the reference's fp8 cache: plain casts, no scales
    view = RaggedPagesCacheView.init(cfg, device=gpu, scaled=True)
    assert tuple(view.kv_scales.shape) == (b.P, 16)
    view.kv_pages.copy_(d["kv_pages"].view(view.kv_pages.shape))
    view.kv_scales.copy_(d["kv_scales"])
    dist = torch.tensor([2, 3, 3], dtype=torch.int32, device=gpu)
    meta = RaggedPagesMetadata(pages_tables=d["block_tables"], context_lens=d["context_lens"], query_start_loc=d["query_start_loc"],
                               num_seqs=d["num_seqs"], request_distribution=dist, page_size=64)
    out = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())(d["query"], None, None, view, meta)
    torch.cuda.synchronize()
    tl.assert_close(tl.from_torch(out.attention_outputs, BF16), tl.oracle_out(b), b, "quantised view")


@pytest.mark.parametrize("name", ["multi_latent_ragged_page_attention_v1", "multi_latent_ragged_page_attention_v2"])
def test_mla_operation_follows_the_model_flow(gpu, name):
    """The layer's flow around the operation (layers/attention/_unified.py:1280-1371): queries absorbed through the key
    half of the up-projection, the operation over latent pages, the output through the value half -- against ordinary
    attention on decompressed keys and values."""
    from easydel_amd.caching import MLARaggedPagesCacheConfig, MLARaggedPagesCacheView

    rng = np.random.default_rng(5)
    heads, lkv, rope, nope, vdim, page_size = 16, 512, 64, 128, 128, 64
    scheduled, computed = [1, 1, 40, 7], [300, 63, 100, 0]
    max_reqs, max_pages = 6, 8
    n_pages = max_reqs * max_pages + 1
    table = np.zeros((max_reqs, max_pages), dtype=np.int32)
    perm = rng.permutation(np.arange(1, n_pages))
    k = 0
    for r in range(len(scheduled)):
        need = -(-(computed[r] + scheduled[r]) // page_size)
        table[r, :need] = perm[k:k + need]
        k += need
    cfg = MLARaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=heads, max_model_length=max_pages * page_size,
                                           kv_lora_rank=lkv, qk_rope_head_dim=rope, page_size=page_size, num_pages=n_pages)
    view = MLARaggedPagesCacheView.init(cfg, layer_index=0, device=gpu)
    assert tuple(view.kv_pages.shape) == (n_pages, page_size // 2, 2, 640)
    sched_full = np.zeros(max_reqs, np.int32); sched_full[:len(scheduled)] = scheduled
    comp_full = np.zeros(max_reqs, np.int32); comp_full[:len(computed)] = computed
    fields = compute_ragged_batch_fields(scheduled_full=sched_full, active_mask_full=sched_full > 0, num_computed_tokens=comp_full,
                                         page_table=table, version="v3", max_num_reqs=max_reqs, page_size=page_size)
    meta = RaggedPagesMetadata.from_numpy(fields, version="v3", page_size=page_size, device=gpu)
    T = int(sum(scheduled))
    bf = lambda a: orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(a.astype(np.float32))).astype(np.float64)  # noqa: E731
    w_k = bf(rng.standard_normal((lkv, heads, nope)) / np.sqrt(lkv))
    w_v = bf(rng.standard_normal((lkv, heads, vdim)) / np.sqrt(lkv))
    q_nope, q_pe = bf(rng.standard_normal((T, heads, nope))), bf(rng.standard_normal((T, heads, rope)))
    latent, k_pe = bf(rng.standard_normal((T, lkv))), bf(rng.standard_normal((T, rope)))
    pool = np.zeros((n_pages, page_size, 640))
    pool[..., :lkv] = bf(rng.standard_normal((n_pages, page_size, lkv)))
    pool[..., 512:576] = bf(rng.standard_normal((n_pages, page_size, rope)))
    view.kv_pages.copy_(torch.from_numpy(pool).to(torch.bfloat16).view(view.kv_pages.shape))
    q_abs = bf(np.einsum("tnd,and->tna", q_nope, w_k))  # the layer casts the absorbed queries back to the model dtype
    tt = lambda a: torch.from_numpy(a).to(torch.bfloat16).to(gpu)  # noqa: E731
    op = OperationRegistry.create(name, OperationMetadata())
    scale = (nope + rope) ** -0.5
    out = op(queries_nope=tt(q_abs)[None], queries_pe=tt(q_pe)[None], keys_values=tt(latent)[None], keys_pe=tt(k_pe)[None],
             cache_view=view, cache_metadata=meta, softmax_scale=scale, causal=True, mask_info=None)
    assert isinstance(out, AttentionOutput) and out.cache_view is view
    assert tuple(out.attention_outputs.shape) == (1, T, heads, lkv)
    got = np.einsum("tna,anh->tnh", out.attention_outputs[0].float().cpu().numpy().astype(np.float64), w_v)
    # the same step through ordinary attention: per-head keys [latent W_k | k_pe] and values latent W_v
    pages = orc.mla_page_scatter_ref(latent, k_pe, pool, fields["context_lens"], table, fields["query_start_loc"],
                                     fields["request_distribution"][2:3])
    np.testing.assert_array_equal(view.kv_pages.view(n_pages, page_size, 640).float().cpu().numpy(), pages)
    d = nope + rope
    dense = np.zeros((n_pages, page_size, 2 * heads, d))
    dense[:, :, 0::2, :nope] = np.einsum("pta,and->ptnd", pages[..., :lkv], w_k)
    dense[:, :, 0::2, nope:] = pages[:, :, None, 512:576]
    dense[:, :, 1::2, :vdim] = np.einsum("pta,anh->ptnh", pages[..., :lkv], w_v)
    want = orc.ragged_paged_attention_ref(np.concatenate([q_nope, q_pe], -1), dense, fields["context_lens"], table,
                                          fields["query_start_loc"], fields["request_distribution"][2:3], softmax_scale=scale,
                                          num_kv_heads=heads)[..., :vdim]
    err = np.abs(got - want)
    # the absorbed queries are rounded to bf16 once more than in the decompressed form; same bars as the kernel tests
    assert err.max() <= tl.TOL_BF16_MAX and err.mean() <= tl.TOL_BF16_MEAN, (err.max(), err.mean())


def test_mla_operation_casts_new_rows_into_an_fp8_latent_cache(gpu):
    """An fp8 latent cache (kvdtype float8_e4m3fn; the cache carries no scales, caching/mla_ragged_page/cache.py:197-204):
    the operation casts the model-dtype rows to the page dtype, the pages then hold the plain cast and attention reads the
    codes' own values."""
    from easydel_amd.caching import MLARaggedPagesCacheConfig, MLARaggedPagesCacheView

    rng = np.random.default_rng(6)
    heads, lkv, rope, page_size = 8, 512, 64, 64
    scheduled, computed = [1, 1, 33], [200, 64, 31]
    max_reqs, max_pages = 4, 4
    n_pages = max_reqs * max_pages + 1
    table = np.zeros((max_reqs, max_pages), dtype=np.int32)
    perm = rng.permutation(np.arange(1, n_pages))
    k = 0
    for r in range(len(scheduled)):
        need = -(-(computed[r] + scheduled[r]) // page_size)
        table[r, :need] = perm[k:k + need]
        k += need
    cfg = MLARaggedPagesCacheConfig.create(torch.float8_e4m3fn, num_hidden_layers=1, num_kv_heads=heads, max_model_length=max_pages * page_size,
                                           kv_lora_rank=lkv, qk_rope_head_dim=rope, page_size=page_size, num_pages=n_pages)
    view = MLARaggedPagesCacheView.init(cfg, layer_index=0, device=gpu)
    assert view.kv_pages.dtype == torch.float8_e4m3fn and tuple(view.kv_pages.shape) == (n_pages, page_size // 4, 4, 640)
    sched_full = np.zeros(max_reqs, np.int32); sched_full[:len(scheduled)] = scheduled
    comp_full = np.zeros(max_reqs, np.int32); comp_full[:len(computed)] = computed
    fields = compute_ragged_batch_fields(scheduled_full=sched_full, active_mask_full=sched_full > 0, num_computed_tokens=comp_full,
                                         page_table=table, version="v3", max_num_reqs=max_reqs, page_size=page_size)
    meta = RaggedPagesMetadata.from_numpy(fields, version="v3", page_size=page_size, device=gpu)
    T = int(sum(scheduled))
    bf = lambda a: orc.bf16_bits_to_f32(orc.f32_to_bf16_bits(a.astype(np.float32))).astype(np.float64)  # noqa: E731
    f8 = lambda a: orc.e4m3fn_bits_to_f32(orc.cast_e4m3fn_ref(a.astype(np.float32))).astype(np.float64)  # noqa: E731
    q_abs, q_pe = bf(rng.standard_normal((T, heads, lkv))), bf(rng.standard_normal((T, heads, rope)))
    latent, k_pe = bf(rng.standard_normal((T, lkv))), bf(rng.standard_normal((T, rope)))
    pool = np.zeros((n_pages, page_size, 640))
    pool[..., :lkv] = f8(rng.standard_normal((n_pages, page_size, lkv)))
    pool[..., 512:576] = f8(rng.standard_normal((n_pages, page_size, rope)))
    codes = orc.cast_e4m3fn_ref(pool.astype(np.float32))
    view.kv_pages.view(torch.uint8).copy_(torch.from_numpy(codes).view(view.kv_pages.shape))
    tt = lambda a: torch.from_numpy(a).to(torch.bfloat16).to(gpu)  # noqa: E731
    op = OperationRegistry.create("multi_latent_ragged_page_attention_v1", OperationMetadata())
    scale = (128 + rope) ** -0.5
    out = op(queries_nope=tt(q_abs)[None], queries_pe=tt(q_pe)[None], keys_values=tt(latent)[None], keys_pe=tt(k_pe)[None],
             cache_view=view, cache_metadata=meta, softmax_scale=scale, causal=True, mask_info=None)
    torch.cuda.synchronize()
    nseq = fields["request_distribution"][2:3]
    pages = orc.mla_page_scatter_ref(f8(latent), f8(k_pe), pool, fields["context_lens"], table, fields["query_start_loc"], nseq)
    got_pages = orc.e4m3fn_bits_to_f32(view.kv_pages.view(torch.uint8).view(n_pages, page_size, 640).cpu().numpy())
    np.testing.assert_array_equal(got_pages, pages)
    want = orc.mla_ragged_paged_attention_ref(q_abs, q_pe, pages, fields["context_lens"], table, fields["query_start_loc"], nseq,
                                              kv_lora_rank=lkv, qk_rope_head_dim=rope, softmax_scale=scale)
    got = out.attention_outputs[0].float().cpu().numpy().astype(np.float64)
    err = np.abs(got - want)[:T]
    big = np.abs(want[:T]) >= 4.0  # a bf16 output there is spaced wider than 2e-2: judged by one bf16 step instead
    bound = np.where(big, 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want[:T]), 1e-30))) - 7), tl.TOL_BF16_MAX)
    assert (err <= np.maximum(bound, tl.TOL_BF16_MAX)).all() and err.mean() <= tl.TOL_BF16_MEAN, (err.max(), err.mean())
