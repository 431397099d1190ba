"""Paged KV cache for the ragged-page attention path: layout, per-layer view, runtime metadata, scatter.

Host-side mirror of the reference's ``easydel/caching/ragged_page/cache.py`` and ``utils.py`` for one
MI355X: the same names, shapes and padding conventions, with torch tensors as the owners of device
memory.  An fp8 cache is by default what it is in the reference: pages of cast codes without scales
(``cache.py:143-158`` gives fp8 a packing of 4; the operation casts K/V to the cache dtype and writes them,
``operations/kernels/ragged_page_attention.py:570-580``).  Two deliberate extensions, both new formats of
this build: int8 is accepted as a cache dtype (the reference's ``get_dtype_packing`` only takes float
dtypes), and a view may carry ``kv_scales [num_pages, combined_heads]`` float32 for fp8-e4m3 / int8 pages
(``RaggedPagesCacheView.init(..., scaled=True)``; always for int8).
"""

from __future__ import annotations

import typing as tp
from dataclasses import dataclass, field

import torch

from .. import kernels

_BITS = {torch.float32: 32, torch.bfloat16: 16, torch.float16: 16, torch.float8_e4m3fn: 8, torch.int8: 8}


def cdiv(a: int, v: int) -> int:
    return (a + v - 1) // v


def align_to_multiple(value: int, multiple: int) -> int:
    return cdiv(value, multiple) * multiple


def get_dtype_packing(dtype) -> int:
    """Elements per 32 bits (reference ``cache.py:143-158``)."""
    bits = _BITS.get(dtype)
    if bits is None:
        raise ValueError(f"unsupported KV cache dtype {dtype}")
    if 32 % bits != 0:
        raise ValueError(f"The bit width must be divisible by 32, but got bits={bits}, dtype={dtype}")
    return 32 // bits


def get_page_size_bytes(page_size: int, num_kv_heads: int, head_size: int, kv_cache_dtype) -> int:
    """Bytes of one page with the storage alignment applied (reference ``cache.py:304-329``)."""
    padded_head_size = cdiv(head_size, 128) * 128
    packing = get_dtype_packing(kv_cache_dtype)
    combined = cdiv(num_kv_heads * 2, packing) * packing
    return page_size * combined * padded_head_size * _BITS[kv_cache_dtype] // 8


@dataclass
class RaggedPagesCacheConfig:
    """Static description of the page pool (reference ``cache.py:374-470``)."""

    num_hidden_layers: int
    max_model_length: int
    num_kv_heads: int
    k_headdim: int
    v_headdim: int
    hbm_utilization: float = 0.9
    data_parallel_size: int = 1
    kv_head_shards: int = 1
    page_size: int = 128
    num_pages: int = -1
    max_num_pages_per_req: int = -1
    version: str = "v3"
    kvdtype: tp.Any = torch.bfloat16

    @classmethod
    def create(cls, kvdtype, num_hidden_layers: int, num_kv_heads: int, max_model_length: int,
               kv_head_dim_size: int | None = None, k_headdim: int | None = None, v_headdim: int | None = None,
               hbm_utilization: float = 0.9, page_size: int = 128, version: str = "v3",
               free_hbm_bytes: int | None = None, num_pages: int | None = None, device="cuda:0",
               mesh=None, partition_manager=None) -> "RaggedPagesCacheConfig":
        """Sizes the pool from free HBM as the reference does (``cache.py:482-594``): one page costs
        ``2 * layers * page_size * num_kv_heads * head_dim * bytes`` and the pool takes
        ``hbm_utilization`` of the free memory.  ``mesh`` / ``partition_manager`` are accepted for call
        compatibility; this build drives one GPU."""
        if k_headdim is None:
            if kv_head_dim_size is None:
                raise ValueError("Either `k_headdim` or `kv_head_dim_size` must be provided")
            k_headdim = kv_head_dim_size
        if v_headdim is None:
            if kv_head_dim_size is None:
                raise ValueError("Either `v_headdim` or `kv_head_dim_size` must be provided")
            v_headdim = kv_head_dim_size
        if num_hidden_layers <= 0:
            raise ValueError("`num_hidden_layers` must be positive")
        if num_kv_heads <= 0:
            raise ValueError("`num_kv_heads` must be positive")
        if k_headdim <= 0 or v_headdim <= 0:
            raise ValueError("`kv_head_dim_size` must be positive")
        if version not in ("v3", "v2"):
            raise ValueError(f"got unknown version {version} it should be v3/v2.")
        get_dtype_packing(kvdtype)
        if num_pages is None:
            if free_hbm_bytes is None:
                free_hbm_bytes, _ = torch.cuda.mem_get_info(device)
            page_bytes = 2 * num_hidden_layers * page_size * num_kv_heads * k_headdim * (_BITS[kvdtype] // 8)
            num_pages = int(free_hbm_bytes * hbm_utilization) // page_bytes
        if num_pages <= 0:
            raise ValueError("Computed `num_pages` is non-positive; increase `hbm_utilization` or reduce page footprint.")
        return cls(num_hidden_layers=num_hidden_layers, max_model_length=max_model_length, num_kv_heads=num_kv_heads,
                   k_headdim=k_headdim, v_headdim=v_headdim, hbm_utilization=hbm_utilization, page_size=page_size,
                   num_pages=num_pages, max_num_pages_per_req=cdiv(max_model_length, page_size), version=version, kvdtype=kvdtype)

    # ---- storage geometry (reference cache.py:606-647) ----
    @property
    def is_v2(self) -> bool:
        return self.version == "v2"

    @property
    def kv_head_packing(self) -> int:
        return get_dtype_packing(self.kvdtype)

    @property
    def storage_num_combined_kv_heads(self) -> int:
        if self.k_headdim == 64:
            return align_to_multiple(self.num_kv_heads, self.kv_head_packing)
        return align_to_multiple(self.num_kv_heads * 2, self.kv_head_packing)

    @property
    def storage_num_kv_groups(self) -> int:
        return self.storage_num_combined_kv_heads // self.kv_head_packing

    @property
    def storage_head_dim(self) -> int:
        if self.k_headdim == 64:
            return 128
        return align_to_multiple(self.k_headdim, 128)

    def get_shape_and_axes(self):
        """``(kv_pages_shape, axes)``; axes are all unsharded on one GPU (reference ``cache.py:695-729``)."""
        if self.version == "v3":
            shape = (self.num_pages, self.page_size, self.storage_num_kv_groups, self.kv_head_packing, self.storage_head_dim)
        elif self.version == "v2":
            shape = (self.num_pages, self.page_size, self.num_kv_heads * 2, self.k_headdim)
        else:
            raise ValueError(f"got unknown version {self.version} it should be v3/v2.")
        return shape, [None] * len(shape)

    @property
    def combined_heads_per_token(self) -> int:
        """Combined K/V heads of ``k_headdim`` elements in one token row of the storage shape."""
        shape, _ = self.get_shape_and_axes()
        per_token = 1
        for s in shape[2:]:
            per_token *= s
        stored = shape[-1]
        if self.k_headdim == 64 and self.version == "v3":
            stored = 64  # K_h | V_h share one 128-wide row
        return per_token // stored


@dataclass
class RaggedPagesMetadata:
    """Per-step metadata (reference ``cache.py:1156-1250``); every array is an int32 device tensor."""

    pages_tables: torch.Tensor  # [max_num_reqs, max_pages]
    context_lens: torch.Tensor  # [max_num_reqs]
    query_start_loc: torch.Tensor  # [max_num_reqs + 1]
    num_seqs: torch.Tensor  # [1] (or longer; element 0 is the count)
    slot_mapping: torch.Tensor | None = None  # v2: [3, num_slices]
    position_ids: torch.Tensor | None = None
    request_distribution: torch.Tensor | None = None  # v3: [decode_end, prefill_end, total]
    num_kv_update_slices: torch.Tensor | None = None  # v2: [1]
    version: str = "v3"
    num_slices_per_kv_cache_update_page: int | None = None
    page_size: int = 128
    prefill_chunk_size: int = 512

    @classmethod
    def create_empty(cls, num_tokens: int, max_num_reqs: int, max_pages: int, page_size: int = 128, version: str = "v3",
                     device="cuda:0") -> "RaggedPagesMetadata":
        z = lambda *shape: torch.zeros(shape, dtype=torch.int32, device=device)  # noqa: E731
        return cls(slot_mapping=z(3, num_tokens) if version == "v2" else None, pages_tables=z(max_num_reqs, max_pages),
                   context_lens=z(max_num_reqs), query_start_loc=z(max_num_reqs + 1), position_ids=z(max_num_reqs),
                   num_seqs=z(max_num_reqs), request_distribution=z(3) if version == "v3" else None,
                   num_kv_update_slices=z(1) if version == "v2" else None, page_size=page_size, version=version)

    @classmethod
    def from_numpy(cls, fields: dict, *, version: str, page_size: int, device="cuda:0") -> "RaggedPagesMetadata":
        """Upload the arrays the host builders of ``easydel_amd.caching.metadata_builder`` return."""
        up = lambda a: None if a is None else torch.as_tensor(a, dtype=torch.int32).to(device)  # noqa: E731
        return cls(pages_tables=up(fields["pages_tables"]), context_lens=up(fields["context_lens"]),
                   query_start_loc=up(fields["query_start_loc"]), num_seqs=up(fields["num_seqs"]),
                   slot_mapping=up(fields.get("slot_mapping")), position_ids=up(fields.get("position_ids")),
                   request_distribution=up(fields.get("request_distribution")),
                   num_kv_update_slices=up(fields.get("num_kv_update_slices")), version=version, page_size=page_size)


def kv_cache_update(new_kv_tokens, slice_indices, kv_cache_pages, total_update_slices, *, page_size: int = 32,
                    page_shard_index: int = 0):
    """In-place paged KV update by slices: the HIP counterpart of ``kv_cache_update_jax``
    (reference ``utils.py:302-387``).  ``kv_cache_pages [total_cache_positions, combined_heads, head_dim]``."""
    return kernels.page_scatter_slices(new_kv_tokens, slice_indices, total_update_slices, kv_cache_pages,
                                       page_size=page_size, page_shard_index=page_shard_index)


@dataclass
class RaggedPagesCacheView:
    """One layer's pages (reference ``cache.py:750-931``)."""

    metadata: RaggedPagesCacheConfig
    kv_pages: torch.Tensor
    layer_index: int | None = None
    kv_scales: torch.Tensor | None = None  # [num_pages, combined_heads] float32 for fp8 / int8 pages

    @classmethod
    def init(cls, config: RaggedPagesCacheConfig, layer_index: int | None = None, device="cuda:0",
             scaled: bool | None = None) -> "RaggedPagesCacheView":
        """Zeroed pages (reference ``cache.py:788-823``).  ``scaled``: give 8-bit pages per-(page, combined head)
        scales, written by the quantising page write; default: only for int8, fp8 pages hold plain casts as in the
        reference."""
        shape, _ = config.get_shape_and_axes()
        pages = torch.zeros(shape, dtype=config.kvdtype, device=device)
        scales = None
        if scaled is None:
            scaled = config.kvdtype == torch.int8
        if scaled:
            if config.kvdtype not in (torch.float8_e4m3fn, torch.int8):
                raise ValueError(f"scaled pages are 8-bit pages, not {config.kvdtype}")
            scales = torch.ones((config.num_pages, config.combined_heads_per_token), dtype=torch.float32, device=device)
        return cls(metadata=config, kv_pages=pages, layer_index=layer_index, kv_scales=scales)

    def concatenate_to_cache(self, key, value, cache_metadata: RaggedPagesMetadata) -> "RaggedPagesCacheView":
        """v2: interleave K/V on the head axis and scatter by ``slot_mapping`` (reference ``cache.py:853-930``);
        v3: nothing to do here, the fused operation writes the pages (``cache.py:931``)."""
        if not self.metadata.is_v2:
            return self
        if self.kv_scales is not None:
            raise NotImplementedError("quantised pages are written by the cache owner, not by concatenate_to_cache")
        num_kv_heads, head_size = key.shape[-2], key.shape[-1]
        key = key.reshape(-1, num_kv_heads, head_size).to(self.kv_pages.dtype)
        value = value.reshape(-1, num_kv_heads, head_size).to(self.kv_pages.dtype)
        kvs = torch.stack([key, value], dim=2).reshape(key.shape[0], 2 * num_kv_heads, head_size).contiguous()
        flat = self.kv_pages.view(-1, *self.kv_pages.shape[2:])
        kv_cache_update(kvs, cache_metadata.slot_mapping, flat, cache_metadata.num_kv_update_slices,
                        page_size=cache_metadata.page_size)
        return self


@dataclass
class RaggedPagesCache:
    """All layers' views (reference ``RaggedPagesCache.init_cache``, ``cache.py:1040-1100``)."""

    views: list = field(default_factory=list)

    @classmethod
    def init_cache(cls, config: RaggedPagesCacheConfig, device="cuda:0") -> "RaggedPagesCache":
        return cls(views=[RaggedPagesCacheView.init(config, layer_index=i, device=device) for i in range(config.num_hidden_layers)])
