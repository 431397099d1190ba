"""CPU tests of the host-side mirror: registry, requirements, cache layout, metadata builders, error paths."""

import logging
from types import SimpleNamespace

import numpy as np
import pytest
import torch

from easydel_amd import caching, kernels
from easydel_amd.caching import RaggedPagesCacheConfig, RaggedPagesCacheView, RaggedPagesMetadata
from easydel_amd.caching import metadata_builder as mb
from easydel_amd.operations import (AttentionOutput, CacheType, ExecutionMode, MetadataField, OperationImpl,
                                    OperationMetadata, OperationRegistry, RaggedPageAttnV2, RaggedPageAttnV3)
from rpa_testlib import orc


def test_registry_names_and_lookup():
    assert OperationRegistry.get("ragged_page_attention_v3") is RaggedPageAttnV3
    assert OperationRegistry.get("ragged_page_attention_v2") is RaggedPageAttnV2
    op = OperationRegistry.create("ragged_page_attention_v3", OperationMetadata())
    assert isinstance(op, RaggedPageAttnV3) and op.get_impl_metadata() is op.metadata
    with pytest.raises(ValueError, match="not found"):
        OperationRegistry.get("no_such_operation")


def test_registry_overwrite_warns_and_replaces(caplog):
    class Fake(OperationImpl):
        @classmethod
        def get_impl_name(cls):
            return ("fake_op_a", "fake_op_b")

        def forward_native(self, *a, **k):
            return "native"

    OperationRegistry.register(Fake)
    with caplog.at_level(logging.WARNING):
        OperationRegistry.register(Fake)
    assert "already registered" in caplog.text
    assert OperationRegistry.get("fake_op_b") is Fake
    assert OperationRegistry.create("fake_op_a", OperationMetadata())() == "native"
    for k in ("fake_op_a", "fake_op_b"):
        OperationRegistry._registry.pop(k)


def test_requirements_declare_ragged_pages_and_exact_view_class():
    for cls, extra in ((RaggedPageAttnV2, MetadataField.SLOT_MAPPING), (RaggedPageAttnV3, MetadataField.REQUEST_DISTRIBUTION)):
        req = cls.get_requirements(ExecutionMode.MIXED)
        assert req.cache.cache_view_class is RaggedPagesCacheView  # the allocator compares by identity
        assert req.cache.is_compatible_with(CacheType.RAGGED_PAGES) and not req.cache.is_compatible_with(CacheType.TRANSFORMER)
        need = MetadataField.SEQ_LENS | MetadataField.CONTEXT_LENS | MetadataField.POSITIONS | MetadataField.QUERY_START_LOC | MetadataField.PAGES_TABLES | extra
        assert req.metadata.required == need and req.metadata.optional == MetadataField.LOGITS_INDICES
        assert req.metadata.is_satisfied_by(need) and not req.metadata.is_satisfied_by(MetadataField.basic())


def test_cache_layout_matches_reference_vectors():
    # tests/layers/caching/test_ragged_page_dtype_compat.py:34-60 of the reference, and cache.py:616-647, 695-729
    cfg = RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=2, num_kv_heads=8, max_model_length=8192,
                                        kv_head_dim_size=128, page_size=64, num_pages=100)
    assert (cfg.kv_head_packing, cfg.storage_num_combined_kv_heads, cfg.storage_num_kv_groups) == (2, 16, 8)
    assert cfg.get_shape_and_axes()[0] == (100, 64, 8, 2, 128) and cfg.max_num_pages_per_req == 128
    cfg8 = RaggedPagesCacheConfig.create(torch.float8_e4m3fn, num_hidden_layers=2, num_kv_heads=4, max_model_length=1024,
                                         kv_head_dim_size=128, num_pages=10)
    assert (cfg8.kv_head_packing, cfg8.storage_num_combined_kv_heads, cfg8.storage_num_kv_groups) == (4, 8, 2)
    c1 = RaggedPagesCacheConfig.create(torch.float32, num_hidden_layers=1, num_kv_heads=2, max_model_length=256,
                                       kv_head_dim_size=64, page_size=16, num_pages=128)
    assert c1.get_shape_and_axes()[0] == (128, 16, 2, 1, 128) and c1.combined_heads_per_token == 4  # K_h|V_h per 128-wide row
    v2 = RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=8, max_model_length=256,
                                       kv_head_dim_size=256, page_size=128, num_pages=4, version="v2")
    assert v2.get_shape_and_axes()[0] == (4, 128, 16, 256) and v2.is_v2
    for tag, (hkv, d, dt) in enumerate([(8, 128, torch.bfloat16), (4, 128, torch.float8_e4m3fn), (2, 64, torch.float32)]):
        c = RaggedPagesCacheConfig.create(dt, num_hidden_layers=1, num_kv_heads=hkv, max_model_length=64, kv_head_dim_size=d, num_pages=2)
        ref = orc.storage_layout_ref(hkv, d, caching.ragged_page._BITS[dt])
        assert (c.kv_head_packing, c.storage_num_combined_kv_heads, c.storage_num_kv_groups, c.storage_head_dim) == \
            (ref["packing"], ref["combined"], ref["groups"], ref["head_dim"])
    assert caching.get_page_size_bytes(64, 8, 128, torch.bfloat16) == 64 * 16 * 128 * 2


def test_cache_config_sizing_and_errors():
    cfg = RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=32, num_kv_heads=8, max_model_length=8192,
                                        kv_head_dim_size=128, page_size=64, hbm_utilization=0.5, free_hbm_bytes=64 << 30)
    page_bytes = 2 * 32 * 64 * 8 * 128 * 2
    assert cfg.num_pages == (32 << 30) // page_bytes
    with pytest.raises(ValueError):
        RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=0, num_kv_heads=8, max_model_length=8, kv_head_dim_size=128, num_pages=1)
    with pytest.raises(ValueError):
        RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=8, max_model_length=8, num_pages=1)
    with pytest.raises(ValueError, match="v3/v2"):
        RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=8, max_model_length=8, kv_head_dim_size=128, num_pages=1, version="v9")
    with pytest.raises(ValueError, match="non-positive"):
        RaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=1, num_kv_heads=8, max_model_length=8, kv_head_dim_size=128, free_hbm_bytes=10)


@pytest.mark.parametrize("scheduled,context_lens,expected", [([4], [4], [0, 1, 1]), ([4, 1, 0], [4, 9, 0], [1, 2, 2])])
def test_request_distribution_reference_vectors(scheduled, context_lens, expected):
    # tests/inference/test_request_distribution_bounds.py:31-44 of the reference
    np.testing.assert_array_equal(mb.request_distribution(scheduled, context_lens), expected)
    from easydel_amd.operations.ragged_page_attention import _request_distribution_bounds

    got = _request_distribution_bounds(torch.tensor(scheduled), torch.tensor(context_lens)).numpy()
    np.testing.assert_array_equal(got, expected)


def test_ragged_batch_fields_reference_vector_and_padding():
    # test_request_distribution_bounds.py:47-58: scheduled [4,1,0,0], computed [0,8,0,0] -> distribution [1,2,2]
    f = mb.compute_ragged_batch_fields(scheduled_full=[4, 1, 0, 0], active_mask_full=[True, True, False, False],
                                       num_computed_tokens=[0, 8, 0, 0], page_table=np.zeros((4, 4), np.int32),
                                       version="v3", max_num_reqs=4)
    np.testing.assert_array_equal(f["request_distribution"], [1, 2, 2])
    np.testing.assert_array_equal(f["query_start_loc"], [0, 4, 5, 5, 5])  # flat extension past the live rows
    np.testing.assert_array_equal(f["context_lens"], [4, 9, 0, 0])
    np.testing.assert_array_equal(f["num_seqs"], [2])
    np.testing.assert_array_equal(f["position_ids"], [0, 1, 2, 3, 8])


def test_slot_mapping_matches_oracle_and_v2_fields():
    rng = np.random.default_rng(0)
    scheduled = np.array([1, 1, 37, 0, 80, 1, 16, 50], dtype=np.int32)
    computed = np.array([5, 15, 0, 9, 3, 31, 16, 100], dtype=np.int32)
    table = rng.permutation(np.arange(1, 81)).reshape(8, 10).astype(np.int32)
    got, total = mb.compute_slot_mapping_v2(num_requests=8, scheduled=scheduled, num_computed_tokens=computed,
                                            page_table=table, page_size=16, slices_per_page=8)
    want, want_total = orc.slot_mapping_v2_ref(scheduled, computed, table, 16, slices_per_page=8)
    np.testing.assert_array_equal(got, want)
    assert total == want_total
    f = mb.compute_ragged_batch_fields(scheduled_full=scheduled, active_mask_full=np.ones(8, bool), num_computed_tokens=computed,
                                       page_table=table, version="v2", max_num_reqs=8, page_size=16, slices_per_page=8)
    np.testing.assert_array_equal(f["slot_mapping"], want)
    np.testing.assert_array_equal(f["num_kv_update_slices"], [want_total])
    assert "request_distribution" not in f
    empty, n = mb.compute_slot_mapping_v2(num_requests=0, scheduled=[], num_computed_tokens=[], page_table=np.zeros((1, 1)), page_size=16)
    assert empty.shape == (3, 1) and n == 0


def test_product_path_refuses_cpu_tensors():
    # there is no CPU fallback: host tensors must raise, not compute
    q = torch.zeros((1, 4, 64), dtype=torch.bfloat16)
    pages = torch.zeros((2, 16, 4, 64), dtype=torch.bfloat16)
    i32 = lambda *v: torch.tensor(v, dtype=torch.int32)  # noqa: E731
    with pytest.raises(RuntimeError, match="GPU memory"):
        kernels.ragged_paged_attention(q, pages, i32(1), i32(1), i32(0, 1), i32(1))
    with pytest.raises(RuntimeError, match="GPU memory"):
        kernels.page_scatter_slices(torch.zeros((1, 4, 64)), torch.zeros((3, 1), dtype=torch.int32), i32(1), torch.zeros((8, 4, 64)), page_size=4)
    view = SimpleNamespace(kv_pages=pages, kv_scales=None, metadata=SimpleNamespace(num_kv_heads=2))
    meta = RaggedPagesMetadata(pages_tables=i32(1).reshape(1, 1), context_lens=i32(1), query_start_loc=i32(0, 1), num_seqs=i32(1),
                               request_distribution=i32(0, 1, 1))
    with pytest.raises(RuntimeError, match="GPU memory"):
        RaggedPageAttnV3(OperationMetadata())(q[None], q[None, :, :2], q[None, :, :2], view, meta)
    with pytest.raises(RuntimeError, match="GPU memory"):
        RaggedPageAttnV3(OperationMetadata())(q[None], q[None, :, :2], q[None, :, :2], view, meta, softmax_aux=torch.zeros(4))
    # attention sinks: one logit per query head, anything else is refused by name
    assert kernels._sinks(None, 4, torch.device("cpu")) == (None, None)
    with pytest.raises(NotImplementedError, match="one sink logit per query head"):
        kernels._sinks(torch.zeros(4, 2), 4, torch.device("cpu"))
    with pytest.raises(NotImplementedError, match="one sink logit per query head"):
        kernels._sinks(torch.zeros(8), 4, torch.device("cpu"))


def test_page_geometry_views():
    assert kernels.page_geometry(torch.empty((5, 64, 16, 128), dtype=torch.bfloat16), 128) == (5, 64, 16, 128)
    assert kernels.page_geometry(torch.empty((5, 64, 8, 2, 128), dtype=torch.bfloat16), 128) == (5, 64, 16, 128)
    assert kernels.page_geometry(torch.empty((5, 16, 2, 1, 128)), 64) == (5, 16, 4, 64)  # v3 storage of head_dim 64: K_h | V_h per row
    # padded head storage (reference cache.py:640-647): head sizes 96 and 192 live in rows of 128 and 256
    assert kernels.page_geometry(torch.empty((5, 16, 4, 2, 128), dtype=torch.bfloat16), 96) == (5, 16, 8, 128)
    assert kernels.page_geometry(torch.empty((5, 16, 2, 4, 256), dtype=torch.float8_e4m3fn), 192) == (5, 16, 8, 256)
    with pytest.raises(ValueError, match="fewer than head_dim"):
        kernels.page_geometry(torch.empty((5, 16, 4, 2, 128), dtype=torch.bfloat16), 192)
    assert kernels.dtype_tag(torch.float16) == 4
    with pytest.raises(NotImplementedError):
        kernels.dtype_tag(torch.float64)


def test_unified_attention_registry_requirements_and_config():
    from easydel_amd.caching import UnifiedAttentionCacheConfig, UnifiedAttentionCacheView
    from easydel_amd.operations import UnifiedAttn

    assert OperationRegistry.get("unified_attention") is UnifiedAttn
    req = UnifiedAttn.get_requirements(ExecutionMode.MIXED)
    assert req.cache.cache_view_class is UnifiedAttentionCacheView and req.cache.is_compatible_with(CacheType.RAGGED_PAGES)
    need = (MetadataField.SEQ_LENS | MetadataField.CONTEXT_LENS | MetadataField.POSITIONS | MetadataField.QUERY_START_LOC
            | MetadataField.PAGES_TABLES | MetadataField.SLOT_MAPPING)
    assert req.metadata.required == need and req.metadata.optional == MetadataField.LOGITS_INDICES
    # sizing: K and V pools of all layers share the budget; slices per update page = min(64, pow2 <= 16 MiB / page bytes)
    cfg = UnifiedAttentionCacheConfig.create(torch.bfloat16, num_hidden_layers=32, num_kv_heads=8, max_model_length=8192,
                                             head_dim=128, page_size=128, hbm_utilization=0.9, free_hbm_bytes=10 << 30)
    assert cfg.num_pages == int((10 << 30) * 0.9) // (2 * 32 * 128 * 8 * 128 * 2)
    assert cfg.version == "v2" and cfg.max_num_pages_per_req == 64 and cfg.num_slices_per_kv_cache_update_page == 32
    assert cfg.get_max_num_seqs() == 1024 * 1024 // 2 // 64 // 4
    assert cfg.get_padded_num_slices(2048, 64) == 160  # 2*64 + 2048/128 = 144, rounded up to a multiple of 32
    assert cfg.get_padded_num_slices(100, 64) == 128   # capped by the token count, then rounded up
    small = UnifiedAttentionCacheConfig.create(torch.bfloat16, 1, 64, 8192, 256, page_size=128, num_pages=3)
    assert small.num_slices_per_kv_cache_update_page == 2  # 16 MiB / 8 MiB pages
    for bad in (dict(num_hidden_layers=0), dict(num_kv_heads=0), dict(head_dim=0), dict(page_size=0), dict(max_model_length=0)):
        kw = dict(num_hidden_layers=1, num_kv_heads=2, max_model_length=64, head_dim=64, page_size=16, num_pages=4)
        kw.update(bad)
        with pytest.raises(ValueError):
            UnifiedAttentionCacheConfig.create(torch.bfloat16, **kw)
    with pytest.raises(ValueError, match="non-positive"):
        UnifiedAttentionCacheConfig.create(torch.bfloat16, 1, 8, 64, 128, free_hbm_bytes=10)


def test_unified_product_path_refuses_cpu_tensors():
    q = torch.zeros((2, 8, 64), dtype=torch.bfloat16)
    pool = torch.zeros((4, 16, 2, 64), dtype=torch.bfloat16)
    i32 = lambda *s: torch.zeros(s, dtype=torch.int32)  # noqa: E731
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        kernels.unified_attention(q, pool, pool.clone(), i32(2), i32(2, 4), i32(3))
    with pytest.raises(ValueError, match="must match"):
        kernels.unified_attention(q, pool, pool[:, :8].contiguous(), i32(2), i32(2, 4), i32(3))


def test_mla_registry_requirements_config_and_errors():
    from easydel_amd.caching import MLARaggedPagesCache, MLARaggedPagesCacheConfig, MLARaggedPagesCacheView
    from easydel_amd.operations import MultiLatentRaggedPageAttn, MultiLatentRaggedPageAttnV2

    assert OperationRegistry.get("multi_latent_ragged_page_attention_v1") is MultiLatentRaggedPageAttn
    assert OperationRegistry.get("multi_latent_ragged_page_attention_v2") is MultiLatentRaggedPageAttnV2
    req = MultiLatentRaggedPageAttnV2.get_requirements(ExecutionMode.MIXED)
    assert req.name == "multi_latent_ragged_page_attention"
    assert req.cache.cache_view_class is MLARaggedPagesCacheView  # the allocator compares view classes by identity
    assert req.metadata.required & MetadataField.REQUEST_DISTRIBUTION and req.cache.is_compatible_with(CacheType.RAGGED_PAGES)

    # sizing rule of caching/mla_ragged_page/cache.py:196-206: a page costs layers * packed tokens * padded row * bytes
    cfg = MLARaggedPagesCacheConfig.create(torch.bfloat16, num_hidden_layers=3, num_kv_heads=128, max_model_length=4096,
                                           kv_lora_rank=512, qk_rope_head_dim=64, page_size=64, free_hbm_bytes=10 * 3 * 64 * 640 * 2,
                                           hbm_utilization=1.0)
    assert cfg.num_pages == 10 and cfg.max_num_pages_per_req == 64 and cfg.version == "v1"
    assert (cfg.kv_lora_rank, cfg.qk_rope_head_dim, cfg.kv_dim, cfg.kv_dim_padded) == (512, 64, 576, 640)
    assert cfg.get_shape_and_axes()[0] == (10, 32, 2, 640)
    # legacy aliases (cache.py:163-171) and the checks of create (:172-194)
    legacy = MLARaggedPagesCacheConfig.create(torch.float32, 1, 1, 128, k_headdim=192, v_headdim=32, page_size=16, num_pages=4)
    assert legacy.kv_dim_padded == 256 + 128 and legacy.get_shape_and_axes()[0] == (4, 16, 1, 384)
    with pytest.raises(ValueError, match="kv_lora_rank"):
        MLARaggedPagesCacheConfig.create(torch.bfloat16, 1, 1, 128, num_pages=4)
    with pytest.raises(ValueError, match="only supports version='v1'"):
        MLARaggedPagesCacheConfig.create(torch.bfloat16, 1, 1, 128, kv_lora_rank=512, version="v3", num_pages=4)
    cache = MLARaggedPagesCache.init_cache(legacy, device="cpu")
    assert len(cache.views) == 1 and cache.metadata is legacy
    view = cache.views[0]
    assert view.key_pages is view.kv_pages and view.value_pages is view.kv_pages and view.concatenate_to_cache(None, None, None) is view

    # argument checks of the operation (multi_latent_ragged_page_attention.py:340-378), before any device work
    op = OperationRegistry.create("multi_latent_ragged_page_attention_v1", OperationMetadata())
    qn, qp = torch.zeros(5, 2, 192), torch.zeros(5, 2, 32)
    kv, pe = torch.zeros(5, 192), torch.zeros(5, 32)
    meta = SimpleNamespace(context_lens=torch.zeros(2, dtype=torch.int32), pages_tables=torch.zeros(2, 8, dtype=torch.int32),
                           query_start_loc=torch.zeros(3, dtype=torch.int32), request_distribution=torch.zeros(3, dtype=torch.int32))
    with pytest.raises(ValueError, match="requires `keys_pe`"):
        op(queries_nope=qn, queries_pe=qp, keys_values=kv, keys_pe=None, cache_view=view, cache_metadata=meta)
    with pytest.raises(ValueError, match="must share"):
        op(queries_nope=qn, queries_pe=qp[:4], keys_values=kv, keys_pe=pe, cache_view=view, cache_metadata=meta)
    with pytest.raises(ValueError, match="token dimension must match"):
        op(queries_nope=qn, queries_pe=qp, keys_values=kv[:3], keys_pe=pe, cache_view=view, cache_metadata=meta)
    with pytest.raises(ValueError, match="rank-3 or rank-4"):
        op(queries_nope=qn[0], queries_pe=qp, keys_values=kv, keys_pe=pe, cache_view=view, cache_metadata=meta)
    with pytest.raises(RuntimeError, match="no CPU fallback"):  # CPU tensors reach the product path and are refused
        op(queries_nope=qn, queries_pe=qp, keys_values=kv, keys_pe=pe, cache_view=view, cache_metadata=meta, unknown_kwarg=1)


def test_mla_distribution_is_derived_on_the_device_when_absent():
    from easydel_amd.operations.multi_latent_ragged_page_attention import _resolve_distribution

    meta = SimpleNamespace(request_distribution=None, query_start_loc=torch.tensor([0, 4, 5, 5], dtype=torch.int32),
                           context_lens=torch.tensor([4, 9, 0], dtype=torch.int32))
    # the second vector of tests/inference/test_request_distribution_bounds.py:30-36
    assert _resolve_distribution(meta).tolist() == [1, 2, 2]
