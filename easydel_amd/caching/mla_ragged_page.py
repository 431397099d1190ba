"""Latent page pool of multi-latent attention (MLA): one row per token, no head axis.

Host-side mirror of the reference's ``easydel/caching/mla_ragged_page/cache.py`` for one GPU: the same
configuration fields, aliases and sizing rule (``MLARaggedPagesCacheConfig.create``, :107-233), the page shape
``[num_pages, page_size / packing, packing, kv_dim_padded]`` (:270-287), a per-layer view whose key and value pages
are the one buffer (:353-384) and the container of all layers' views (:395-450).  The arrays are torch tensors in
GPU memory.  The pages are written by the attention operation itself (the fused call); the view's
``concatenate_to_cache`` therefore has nothing to do, as in the reference, whose view inherits the v3 behaviour.
"""

from __future__ import annotations

import typing as tp
from dataclasses import dataclass, field

import torch

from .ragged_page import _BITS, align_to_multiple, cdiv, get_dtype_packing


@dataclass
class MLARaggedPagesCacheConfig:
    """Static description of the latent pool.  ``k_headdim`` holds ``kv_lora_rank`` and ``v_headdim`` holds
    ``qk_rope_head_dim``, the reference's legacy aliases (:149-151, 221-222)."""

    num_hidden_layers: int
    max_model_length: int
    num_kv_heads: int
    k_headdim: int
    v_headdim: int
    hbm_utilization: float = 0.9
    data_parallel_size: int = 1
    page_size: int = 128
    num_pages: int = -1
    max_num_pages_per_req: int = -1
    version: str = "v1"
    kvdtype: tp.Any = torch.bfloat16

    @classmethod
    def create(cls, kvdtype, num_hidden_layers: int, num_kv_heads: int, max_model_length: int, *,
               kv_lora_rank: int | None = None, qk_rope_head_dim: int | None = None, kv_head_dim_size: int | None = None,
               k_headdim: int | None = None, v_headdim: int | None = None, hbm_utilization: float = 0.9,
               page_size: int = 128, version: str = "v1", free_hbm_bytes: int | None = None, num_pages: int | None = None,
               device="cuda:0", mesh=None, partition_manager=None) -> "MLARaggedPagesCacheConfig":
        """Sizes the pool as the reference does (:163-233): a page costs
        ``layers * packed_page_tokens * kv_dim_padded * bytes`` and the pool takes ``hbm_utilization`` of the free
        memory.  ``mesh`` / ``partition_manager`` are accepted for call compatibility; this build drives one GPU."""
        if kv_lora_rank is None:
            kv_lora_rank = k_headdim
        if qk_rope_head_dim is None:
            qk_rope_head_dim = v_headdim
        if kv_lora_rank is None and kv_head_dim_size is not None:
            kv_lora_rank = kv_head_dim_size
        if qk_rope_head_dim is None:
            qk_rope_head_dim = 0
        if num_hidden_layers <= 0:
            raise ValueError("`num_hidden_layers` must be positive")
        if num_kv_heads <= 0:
            raise ValueError("`num_kv_heads` must be positive")
        if max_model_length <= 0:
            raise ValueError("`max_model_length` must be positive")
        if kv_lora_rank is None or kv_lora_rank <= 0:
            raise ValueError("`kv_lora_rank` must be positive")
        if qk_rope_head_dim < 0:
            raise ValueError("`qk_rope_head_dim` must be non-negative")
        if page_size <= 0:
            raise ValueError("`page_size` must be positive")
        if version != "v1":
            raise ValueError(f"MLA ragged cache only supports version='v1', got {version!r}")
        packing = get_dtype_packing(kvdtype)
        if num_pages is None:
            if free_hbm_bytes is None:
                free_hbm_bytes, _ = torch.cuda.mem_get_info(device)
            kv_dim_padded = align_to_multiple(int(kv_lora_rank), 128) + align_to_multiple(int(qk_rope_head_dim), 128)
            packed_page_tokens = cdiv(page_size, packing) * packing
            page_bytes = num_hidden_layers * packed_page_tokens * kv_dim_padded * (_BITS[kvdtype] // 8)
            num_pages = int(free_hbm_bytes * hbm_utilization) // page_bytes
        if num_pages <= 0:
            raise ValueError("Computed `num_pages` is non-positive; increase `hbm_utilization` or reduce page footprint.")
        return cls(num_hidden_layers=num_hidden_layers, max_model_length=max_model_length, num_kv_heads=num_kv_heads,
                   k_headdim=int(kv_lora_rank), v_headdim=int(qk_rope_head_dim), hbm_utilization=hbm_utilization,
                   page_size=page_size, num_pages=num_pages, max_num_pages_per_req=cdiv(max_model_length, page_size),
                   version="v1", kvdtype=kvdtype)

    # ---- geometry (reference :235-287) ----
    @property
    def kv_lora_rank(self) -> int:
        return int(self.k_headdim)

    @property
    def qk_rope_head_dim(self) -> int:
        return int(self.v_headdim)

    @property
    def kv_dim(self) -> int:
        return self.kv_lora_rank + self.qk_rope_head_dim

    @property
    def kv_dim_padded(self) -> int:
        return align_to_multiple(self.kv_lora_rank, 128) + align_to_multiple(self.qk_rope_head_dim, 128)

    @property
    def kv_packing(self) -> int:
        return get_dtype_packing(self.kvdtype)

    @property
    def page_size_per_kv_packing(self) -> int:
        return cdiv(int(self.page_size), int(self.kv_packing))

    def get_shape_and_axes(self):
        shape = (int(self.num_pages), self.page_size_per_kv_packing, self.kv_packing, self.kv_dim_padded)
        return shape, ("attn_dp", None, None, None)


@dataclass
class MLARaggedPagesCacheView:
    """One layer's latent pages (reference :290-392)."""

    metadata: MLARaggedPagesCacheConfig
    kv_pages: torch.Tensor
    layer_index: int | None = None

    @classmethod
    def init(cls, config: MLARaggedPagesCacheConfig, layer_index: int | None = None, device="cuda:0", mesh=None,
             partition_manager=None, quantizer=None) -> "MLARaggedPagesCacheView":
        if quantizer is not None:
            raise NotImplementedError("quantised latent pages are not supported")
        shape, _ = config.get_shape_and_axes()
        return cls(metadata=config, kv_pages=torch.zeros(shape, dtype=config.kvdtype, device=device), layer_index=layer_index)

    def flattened_kv_pages(self) -> torch.Tensor:
        return self.kv_pages

    @property
    def key_pages(self) -> torch.Tensor:
        return self.flattened_kv_pages()

    @property
    def value_pages(self) -> torch.Tensor:
        return self.flattened_kv_pages()

    def concatenate_to_cache(self, *args, **kwargs) -> "MLARaggedPagesCacheView":
        """Nothing to do: the attention operation writes the new rows itself."""
        return self


@dataclass
class MLARaggedPagesCache:
    """All layers' views (reference :395-450)."""

    views: list = field(default_factory=list)

    @property
    def metadata(self) -> MLARaggedPagesCacheConfig | None:
        if not self.views or self.views[-1] is None:
            return None
        return self.views[-1].metadata

    @classmethod
    def init_cache(cls, config: MLARaggedPagesCacheConfig, device="cuda:0", mesh=None, partition_manager=None,
                   quantizer=None) -> "MLARaggedPagesCache":
        return cls(views=[MLARaggedPagesCacheView.init(config, layer_index=i, device=device, quantizer=quantizer)
                          for i in range(config.num_hidden_layers)])
