"""Unified-attention paged KV cache: separate K and V pools ``[num_pages, page_size, num_kv_heads, head_dim]``.

Host-side mirror of the reference's ``easydel/caching/unified_attention/cache.py`` for one GPU: the same
configuration fields and sizing rules (``UnifiedAttentionCacheConfig.create``, :299-386; padded slice count,
:399-426; sequence heuristic, :428-441), a per-layer view whose ``concatenate_to_cache`` writes new K and V with
the v2 slot mapping (:523-610), and the container of all layers' views (:623-704).  The arrays are torch tensors
in GPU memory; the writes go through the slice-scatter entry point of ``librpa_hip.so``.
"""

from __future__ import annotations

import typing as tp
from dataclasses import dataclass, field

import torch

from .ragged_page import _BITS, RaggedPagesMetadata, cdiv, kv_cache_update


def _previous_power_of_2(n: int) -> int:
    """Largest power of two <= n, and 1 for n <= 1 (reference :143-154)."""
    if n <= 1:
        return 1
    return 1 << (int(n).bit_length() - 1)


@dataclass
class UnifiedAttentionCacheConfig:
    """Static description of the two pools (reference :209-272)."""

    num_hidden_layers: int
    max_model_length: int
    num_kv_heads: int
    head_dim: int
    hbm_utilization: float = 0.9
    data_parallel_size: int = 1
    page_size: int = 128
    num_pages: int = -1
    max_num_pages_per_req: int = -1
    window_aware_max_num_seqs: int = -1
    window_aware_pages_per_request: int = -1
    window_aware_max_num_batched_tokens: int = -1
    num_slices_per_kv_cache_update_page: int = -1
    version: str = "v2"  # the pools are filled with the v2 slot mapping
    kvdtype: tp.Any = torch.bfloat16

    @classmethod
    def create(cls, kvdtype, num_hidden_layers: int, num_kv_heads: int, max_model_length: int, head_dim: int, *,
               hbm_utilization: float = 0.9, page_size: int = 128, free_hbm_bytes: int | None = None,
               num_pages: int | None = None, device="cuda:0", mesh=None, partition_manager=None
               ) -> "UnifiedAttentionCacheConfig":
        """Sizes the pools as the reference does (:344-386): a page costs
        ``2 * layers * page_size * num_kv_heads * head_dim * bytes`` (K and V) and the pools take
        ``hbm_utilization`` of the free memory.  ``mesh`` / ``partition_manager`` are accepted for call
        compatibility; this build drives one GPU."""
        if num_hidden_layers <= 0:
            raise ValueError("`num_hidden_layers` must be positive")
        if num_kv_heads <= 0:
            raise ValueError("`num_kv_heads` must be positive")
        if head_dim <= 0:
            raise ValueError("`head_dim` must be positive")
        if page_size <= 0:
            raise ValueError("`page_size` must be positive")
        if max_model_length <= 0:
            raise ValueError("`max_model_length` must be positive")
        bytes_av = _BITS[kvdtype] // 8
        if num_pages is None:
            if free_hbm_bytes is None:
                free_hbm_bytes, _ = torch.cuda.mem_get_info(device)
            page_bytes = 2 * num_hidden_layers * page_size * num_kv_heads * head_dim * bytes_av
            num_pages = int(free_hbm_bytes * hbm_utilization) // page_bytes
        if num_pages <= 0:
            raise ValueError("Computed `num_pages` is non-positive; increase `hbm_utilization` or reduce page footprint.")
        page_size_bytes = 2 * page_size * num_kv_heads * head_dim * bytes_av
        slices_raw = (16 * 1024 * 1024) // max(1, int(page_size_bytes))
        return cls(num_hidden_layers=num_hidden_layers, max_model_length=max_model_length, num_kv_heads=num_kv_heads,
                   head_dim=head_dim, hbm_utilization=hbm_utilization, page_size=page_size, num_pages=int(num_pages),
                   max_num_pages_per_req=cdiv(max_model_length, page_size),
                   num_slices_per_kv_cache_update_page=int(min(64, _previous_power_of_2(int(slices_raw)))), kvdtype=kvdtype)

    def get_padded_num_slices(self, num_tokens: int | None = None, max_num_reqs: int | None = None) -> int:
        """Slice-count bound of one cache update, rounded up to the slices-per-page unit (reference :399-426)."""
        if num_tokens is None or num_tokens <= 0:
            num_tokens = self.max_model_length
        if max_num_reqs is None or max_num_reqs <= 0:
            max_num_reqs = self.get_max_num_seqs()
        padded = 2 * int(max_num_reqs) + int(num_tokens) // int(self.page_size)
        padded = min(int(padded), int(num_tokens))
        unit = max(1, int(self.num_slices_per_kv_cache_update_page))
        return int(((padded + unit - 1) // unit) * unit)

    def get_max_num_seqs(self) -> int:
        """Reference :428-441."""
        if self.window_aware_max_num_seqs > 0:
            return int(self.window_aware_max_num_seqs)
        return 1024 * 1024 // 2 // cdiv(self.max_model_length, self.page_size) // 4


@dataclass
class UnifiedAttentionCacheView:
    """One layer's K pool and V pool (reference :445-620)."""

    metadata: UnifiedAttentionCacheConfig
    key_cache: torch.Tensor
    value_cache: torch.Tensor
    layer_index: int = 0

    @classmethod
    def init(cls, config: UnifiedAttentionCacheConfig, layer_index: int | None = None, device="cuda:0",
             mesh=None, partition_manager=None, quantizer=None) -> "UnifiedAttentionCacheView":
        if quantizer is not None:
            raise NotImplementedError("a quantizer for the unified-attention pools is not part of this build")
        shape = (config.num_pages, config.page_size, config.num_kv_heads, config.head_dim)
        return cls(metadata=config, key_cache=torch.zeros(shape, dtype=config.kvdtype, device=device),
                   value_cache=torch.zeros(shape, dtype=config.kvdtype, device=device), layer_index=layer_index or 0)

    def concatenate_to_cache(self, key, value, cache_metadata: RaggedPagesMetadata) -> "UnifiedAttentionCacheView":
        """Writes the step's new K and V rows into their pools by ``slot_mapping`` (reference :523-610): the same
        slice scatter as the interleaved v2 cache, run once per pool on rows of ``num_kv_heads * head_dim``."""
        if cache_metadata.slot_mapping is None or cache_metadata.num_kv_update_slices is None:
            raise ValueError("UnifiedAttentionCacheView requires v2-style `slot_mapping` and `num_kv_update_slices`.")
        key_tokens = key.reshape(-1, *key.shape[-2:]).to(self.key_cache.dtype).contiguous()
        value_tokens = value.reshape(-1, *value.shape[-2:]).to(self.value_cache.dtype).contiguous()
        for tokens, pool in ((key_tokens, self.key_cache), (value_tokens, self.value_cache)):
            kv_cache_update(tokens, cache_metadata.slot_mapping, pool.view(-1, *pool.shape[2:]),
                            cache_metadata.num_kv_update_slices, page_size=int(cache_metadata.page_size))
        return self

    def __repr__(self) -> str:
        return (f"{self.__class__.__name__}(layer_index={self.layer_index}, "
                f"key_cache_shape={tuple(self.key_cache.shape)}, value_cache_shape={tuple(self.value_cache.shape)})")


@dataclass
class UnifiedAttentionCache:
    """All layers' views (reference :623-704)."""

    views: list = field(default_factory=list)

    @classmethod
    def init_cache(cls, config: UnifiedAttentionCacheConfig, device="cuda:0", mesh=None, partition_manager=None,
                   quantizer=None) -> "UnifiedAttentionCache":
        return cls(views=[UnifiedAttentionCacheView.init(config, layer_index=i, device=device, quantizer=quantizer)
                          for i in range(config.num_hidden_layers)])

    @classmethod
    def init_empty(cls, num_hidden_layers: int, *args, **kwargs) -> "UnifiedAttentionCache":
        return cls(views=[None for _ in range(num_hidden_layers)])
