from .metadata_builder import compute_ragged_batch_fields, compute_slot_mapping_v2, request_distribution
from .ragged_page import (
    RaggedPagesCache,
    RaggedPagesCacheConfig,
    RaggedPagesCacheView,
    RaggedPagesMetadata,
    get_dtype_packing,
    get_page_size_bytes,
    kv_cache_update,
)
from .mla_ragged_page import MLARaggedPagesCache, MLARaggedPagesCacheConfig, MLARaggedPagesCacheView
from .unified_attention import UnifiedAttentionCache, UnifiedAttentionCacheConfig, UnifiedAttentionCacheView

__all__ = [
    "MLARaggedPagesCache", "MLARaggedPagesCacheConfig", "MLARaggedPagesCacheView",
    "UnifiedAttentionCache", "UnifiedAttentionCacheConfig", "UnifiedAttentionCacheView",
    "RaggedPagesCache", "RaggedPagesCacheConfig", "RaggedPagesCacheView", "RaggedPagesMetadata", "get_dtype_packing",
    "get_page_size_bytes", "kv_cache_update", "compute_ragged_batch_fields", "compute_slot_mapping_v2", "request_distribution",
]
