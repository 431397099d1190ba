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
    view = RaggedPagesCacheView.init(cfg, device=gpu)
    assert tuple(view.kv_scales.shape) == (b.P, 16)
    view.kv_pages.copy_(d["kv_pages"].view(view.kv_pages.shape))
    view.kv_scales.copy_(d["kv_scales"])
    dist = torch.tensor([2, 3, 3], dtype=torch.int32, device=gpu)
    meta = RaggedPagesMetadata(pages_tables=d["block_tables"], context_lens=d["context_lens"], query_start_loc=d["query_start_loc"],
                               num_seqs=d["num_seqs"], request_distribution=dist, page_size=64)
    out = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())(d["query"], None, None, view, meta)
    torch.cuda.synchronize()
    tl.assert_close(tl.from_torch(out.attention_outputs, BF16), tl.oracle_out(b), b, "quantised view")
