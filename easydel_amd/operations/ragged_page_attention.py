"""``ragged_page_attention_v2`` / ``_v3`` operations backed by the MI355X HIP kernels.

Drop-in for the reference's ``easydel/operations/kernels/ragged_page_attention.py``: the same class names,
registry names, call signature (``query, key, value, cache_view, cache_metadata, softmax_scale,
logits_soft_cap, sliding_window`` plus swallowed extras), 4-D <-> ragged reshape (:881-918), cast of K/V to
the cache dtype with a warning when it narrows (:570-580), write-back of the updated pages into the view
(:747), ``softmax_aux`` attention sinks (one logit per query head, cast to float32 as at :469-471) and
``AttentionOutput`` result.  Where the reference hands the arrays to ``ejkernel`` (:281-313,
:732-746), this module hands device pointers to ``librpa_hip.so`` through ``easydel_amd.kernels``.
"""

from __future__ import annotations

import logging

import torch

from .. import kernels
from ..caching.ragged_page import RaggedPagesCacheView, RaggedPagesMetadata
from ._attention_outputs import AttentionOutput
from ._base_operation import OperationImpl, OperationRegistry
from .requirements import CacheType, ExecutionMode, MetadataField, OperationRequirements, RequirementsBuilder

logger = logging.getLogger(__name__)


def _request_distribution_bounds(scheduled: torch.Tensor, context_lens: torch.Tensor) -> torch.Tensor:
    """``[decode_end, prefill_end, total]`` on the device (reference :177-187)."""
    scheduled = scheduled.to(torch.int32)
    context_lens = context_lens.to(torch.int32)
    has_tokens = scheduled > 0
    is_decode = (scheduled == 1) & (context_lens > 1) & has_tokens
    decode = is_decode.sum()
    prefill = (has_tokens & ~is_decode).sum()
    return torch.stack((decode, decode + prefill, has_tokens.sum())).to(torch.int32)


def dp_local_metadata(cache_metadata, shard_index: int, num_shards: int, local_pages: int):
    """``(context_lens, flat block tables, query_start_loc, distribution)`` of one data-parallel rank when the page pool
    is sharded over ranks (reference :650-681; the same lines serve the multi-latent operation,
    multi_latent_ragged_page_attention.py:507-536): the rank's rows of the lengths and page tables, the matching
    ``rows + 1`` entries of ``query_start_loc`` (token indices stay global), the request distribution recomputed for them,
    page ids rebased by ``shard_index * local_pages`` and clipped into the local pool.  All on the device."""
    S = int(cache_metadata.context_lens.shape[0])
    if num_shards <= 0 or S % num_shards != 0:
        raise ValueError(f"{S} metadata rows do not divide over {num_shards} shards")  # the reference falls back to the global path
    if not 0 <= shard_index < num_shards:
        raise ValueError(f"shard_index {shard_index} outside [0, {num_shards})")
    rows = S // num_shards
    row_start = shard_index * rows
    max_pages = int(cache_metadata.pages_tables.numel()) // S
    context_lens = cache_metadata.context_lens[row_start:row_start + rows].contiguous()
    tables = cache_metadata.pages_tables.reshape(S, max_pages)[row_start:row_start + rows]
    query_start_loc = cache_metadata.query_start_loc[row_start:row_start + rows + 1].contiguous()
    distribution = _request_distribution_bounds(query_start_loc[1:] - query_start_loc[:-1], context_lens)
    tables = (tables - shard_index * local_pages).clamp(0, local_pages - 1).to(torch.int32).reshape(-1).contiguous()
    return context_lens, tables, query_start_loc, distribution


class _RaggedPageAttn(OperationImpl):
    """Attention over a paged KV cache for ragged batches (prefill, chunked prefill and decode rows mixed)."""

    @classmethod
    def get_impl_name(cls) -> str | tuple[str]:
        raise NotImplementedError()

    # -- v2: read-only attention over pages the cache view already updated ------------------------------
    def forward_v2(self, query, cache_view: RaggedPagesCacheView, cache_metadata: RaggedPagesMetadata,
                   softmax_scale: float | None = None, logits_soft_cap: float | None = None, compute_dtype=None,
                   optimized: bool = False, sliding_window: int | None = None, softmax_aux=None,
                   mask_value: float | None = None, vmem_limit_bytes: int | None = None, **ignore) -> AttentionOutput:
        output = kernels.ragged_paged_attention(
            query, cache_view.kv_pages, cache_metadata.context_lens, cache_metadata.pages_tables,
            cache_metadata.query_start_loc, cache_metadata.num_seqs.reshape(-1), softmax_scale=softmax_scale,
            sliding_window=sliding_window, logits_soft_cap=logits_soft_cap,
            kv_scales=getattr(cache_view, "kv_scales", None), num_kv_heads=_num_kv_heads(cache_view),
            softmax_aux=softmax_aux)
        return AttentionOutput(attention_weights=None, attention_outputs=output)

    # -- v3: fused page write + attention ------------------------------------------------------------------
    def forward_v3(self, query, key, value, cache_view: RaggedPagesCacheView, cache_metadata: RaggedPagesMetadata,
                   softmax_scale: float | None = None, logits_soft_cap: float | None = None,
                   sliding_window: int | None = None, softmax_aux=None, **ignore) -> AttentionOutput:
        kv_pages = cache_view.kv_pages
        if getattr(cache_view, "kv_scales", None) is not None:
            # scaled 8-bit pages: the write quantises (per page and head the scale only grows), then the attention
            # reads codes and scales
            if key is None or value is None:  # nothing to write: read the pages as they are
                output = kernels.ragged_paged_attention(
                    query, kv_pages, cache_metadata.context_lens, cache_metadata.pages_tables.reshape(-1),
                    cache_metadata.query_start_loc, cache_metadata.request_distribution[2:3], softmax_scale=softmax_scale,
                    sliding_window=sliding_window, logits_soft_cap=logits_soft_cap, kv_scales=cache_view.kv_scales,
                    num_kv_heads=_num_kv_heads(cache_view), softmax_aux=softmax_aux)
                return AttentionOutput(attention_weights=None, attention_outputs=output, cache_view=cache_view)
            if key.dtype not in (torch.float32, torch.bfloat16):
                key, value = key.to(torch.float32), value.to(torch.float32)
            output, kv_pages, kv_scales = kernels.ragged_paged_attention_v3_quantised(
                query, key.contiguous(), value.to(key.dtype).contiguous(), kv_pages, cache_view.kv_scales,
                cache_metadata.context_lens, cache_metadata.pages_tables.reshape(-1), cache_metadata.query_start_loc,
                cache_metadata.request_distribution, softmax_scale=softmax_scale, sliding_window=sliding_window,
                logits_soft_cap=logits_soft_cap, num_kv_heads=_num_kv_heads(cache_view), softmax_aux=softmax_aux)
            cache_view.kv_pages, cache_view.kv_scales = kv_pages, kv_scales
            return AttentionOutput(attention_weights=None, attention_outputs=output, cache_view=cache_view)
        if key.dtype != kv_pages.dtype or value.dtype != kv_pages.dtype:
            if kv_pages.element_size() < max(key.element_size(), value.element_size()):
                logger.warning("Casting key/value from %s to lower-precision KV cache dtype %s; "
                               "this may reduce numerical fidelity.", key.dtype, kv_pages.dtype)
            key = key.to(kv_pages.dtype)
            value = value.to(kv_pages.dtype)
        output, kv_pages = kernels.ragged_paged_attention_v3(
            query, key.contiguous(), value.contiguous(), kv_pages, cache_metadata.context_lens,
            cache_metadata.pages_tables.reshape(-1), cache_metadata.query_start_loc, cache_metadata.request_distribution,
            softmax_scale=softmax_scale, sliding_window=sliding_window, logits_soft_cap=logits_soft_cap,
            softmax_aux=softmax_aux)
        cache_view.kv_pages = kv_pages
        return AttentionOutput(attention_weights=None, attention_outputs=output, cache_view=cache_view)

    # -- v3 on pages sharded over data-parallel ranks: one rank's share ------------------------------------------
    def forward_v3_dp_local_shard(self, query, key, value, local_kv_pages, cache_metadata: RaggedPagesMetadata,
                                  shard_index: int, num_shards: int, softmax_scale: float | None = None,
                                  logits_soft_cap: float | None = None, sliding_window: int | None = None,
                                  softmax_aux=None, local_kv_scales=None, num_kv_heads: int | None = None, **ignore):
        """What one data-parallel rank computes when the page pool is sharded over ranks and every sequence's pages
        live on the rank that owns its metadata row (the body of the reference's ``shard_map`` at :645-717, before the
        sum over ranks): the rank takes its ``S / num_shards`` rows of ``context_lens``, ``pages_tables`` and
        ``query_start_loc`` (token indices stay global: every rank holds the whole query), recomputes the request
        distribution for them, rebases the page ids by ``shard_index * local_pages`` and clips them into the local
        pool, runs the fused write + attention on its pages, and returns output rows that are zero for the tokens of
        other ranks' sequences.  Returns ``(local_output, local_kv_pages)``; the ranks' outputs are then summed in
        float32 (:699-717) -- ``dp_local_reduce`` does that for outputs gathered on one device.  Nothing here reads
        device values on the host.

        A rank's share of a scaled 8-bit pool comes with its rows of the scales, ``local_kv_scales [local_pages, C]``:
        the write then quantises and the call returns ``(local_output, local_kv_pages, local_kv_scales)``.  int8 pages
        without scales are refused (only fp8 pages may hold bare codes, the reference's cast-only cache)."""
        context_lens, tables, query_start_loc, distribution = dp_local_metadata(cache_metadata, shard_index, num_shards, int(local_kv_pages.shape[0]))
        if local_kv_scales is not None:
            if key.dtype not in (torch.float32, torch.bfloat16):
                key, value = key.to(torch.float32), value.to(torch.float32)
            return kernels.ragged_paged_attention_v3_quantised(
                query, key.contiguous(), value.to(key.dtype).contiguous(), local_kv_pages, local_kv_scales, context_lens, tables,
                query_start_loc, distribution, softmax_scale=softmax_scale, sliding_window=sliding_window,
                logits_soft_cap=logits_soft_cap, num_kv_heads=num_kv_heads, softmax_aux=softmax_aux)
        if local_kv_pages.dtype == torch.int8:
            raise ValueError("int8 KV pages are always scaled: pass this rank's rows of the scales as local_kv_scales")
        if key.dtype != local_kv_pages.dtype or value.dtype != local_kv_pages.dtype:
            key, value = key.to(local_kv_pages.dtype), value.to(local_kv_pages.dtype)
        # tokens outside [query_start_loc[0], query_start_loc[total]) belong to other ranks: the kernels write zeros
        # for them, which is the masking of :699-712
        return kernels.ragged_paged_attention_v3(
            query, key.contiguous(), value.contiguous(), local_kv_pages, context_lens, tables, query_start_loc, distribution,
            softmax_scale=softmax_scale, sliding_window=sliding_window, logits_soft_cap=logits_soft_cap, softmax_aux=softmax_aux)

    def forward_native(self, query, key, value, cache_view, cache_metadata, softmax_scale: float | None = None,
                       logits_soft_cap: float | None = None, sliding_window: int | None = None, softmax_aux=None,
                       vmem_limit_bytes: int | None = None, mask_value: float | None = None, compute_dtype=None,
                       optimized: bool = False, **ignore):
        fn = self.forward_v3 if self.get_impl_name() == "ragged_page_attention_v3" else self.forward_v2
        return fn(query=query, key=key, value=value, cache_view=cache_view, cache_metadata=cache_metadata,
                  softmax_scale=softmax_scale, logits_soft_cap=logits_soft_cap, vmem_limit_bytes=vmem_limit_bytes,
                  optimized=optimized, compute_dtype=compute_dtype, softmax_aux=softmax_aux, mask_value=mask_value,
                  sliding_window=sliding_window, **ignore)

    def forward_gpu(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)

    def forward_rocm(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)

    def __call__(self, query, key, value, cache_view, cache_metadata, softmax_scale: float | None = None,
                 logits_soft_cap: float | None = None, compute_dtype=None, optimized: bool = False,
                 sliding_window: int | None = None, softmax_aux=None, mask_value: float | None = None,
                 vmem_limit_bytes: int | None = None, **ignore) -> AttentionOutput:
        is_4d = query.ndim == 4
        shape4 = tuple(query.shape) if is_4d else None
        query_r = query.reshape(-1, *query.shape[-2:]).contiguous()
        key_r = None if key is None else key.reshape(-1, *key.shape[-2:])
        value_r = None if value is None else value.reshape(-1, *value.shape[-2:])
        output = super().__call__(query=query_r, key=key_r, value=value_r, cache_view=cache_view,
                                  cache_metadata=cache_metadata, softmax_scale=softmax_scale,
                                  logits_soft_cap=logits_soft_cap, vmem_limit_bytes=vmem_limit_bytes, optimized=optimized,
                                  compute_dtype=compute_dtype, softmax_aux=softmax_aux, mask_value=mask_value,
                                  sliding_window=sliding_window, **ignore)
        if is_4d:
            output.attention_outputs = output.attention_outputs.reshape(shape4)
        return output


def dp_local_reduce(local_outputs) -> torch.Tensor:
    """The sum over data-parallel ranks the reference performs on the shard outputs: in float32, cast back to the output
    dtype (:713-717).  For outputs that already sit on one device; across GPUs it is an all-reduce of the same values."""
    total = local_outputs[0].to(torch.float32)
    for other in local_outputs[1:]:
        total = total + other.to(torch.float32)
    return total.to(local_outputs[0].dtype)


def _num_kv_heads(cache_view) -> int | None:
    meta = getattr(cache_view, "metadata", None)
    n = getattr(meta, "num_kv_heads", None)
    return int(n) if n else None


def _requirements(name: str, extra: MetadataField) -> OperationRequirements:
    return (RequirementsBuilder(name)
            .require_metadata(MetadataField.SEQ_LENS | MetadataField.CONTEXT_LENS | MetadataField.POSITIONS
                              | MetadataField.QUERY_START_LOC | MetadataField.PAGES_TABLES | extra)
            .optional_metadata(MetadataField.LOGITS_INDICES)
            .support_cache(CacheType.RAGGED_PAGES)
            .use_cache_view(RaggedPagesCacheView)
            .build())


@OperationRegistry.register
class RaggedPageAttnV2(_RaggedPageAttn):
    @classmethod
    def get_impl_name(cls) -> str | tuple[str]:
        return "ragged_page_attention_v2"

    @classmethod
    def get_requirements(cls, mode: ExecutionMode = ExecutionMode.MIXED) -> OperationRequirements:
        return _requirements("ragged_page_attention_v2", MetadataField.SLOT_MAPPING)


@OperationRegistry.register
class RaggedPageAttnV3(_RaggedPageAttn):
    @classmethod
    def get_impl_name(cls) -> str | tuple[str]:
        return "ragged_page_attention_v3"

    @classmethod
    def get_requirements(cls, mode: ExecutionMode = ExecutionMode.MIXED) -> OperationRequirements:
        return _requirements("ragged_page_attention_v3", MetadataField.REQUEST_DISTRIBUTION)
