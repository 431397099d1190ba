"""``unified_attention`` operation (separate K and V pools) backed by the MI355X HIP kernels.

Drop-in for the reference's ``easydel/operations/kernels/unified_attention.py``: the same class and registry
name (:84, :113), requirements (:117-147), call signature of ``forward_native`` (:149-160), 4-D <-> ragged
reshape (:256-262, :395-396) and ``AttentionOutput`` result.  Where the reference hands the arrays to
``ejkernel.modules.unified_attention`` (:363-388) this module hands device pointers to ``librpa_hip.so``.  The
operation reads the pools only: the step's K/V are written before by the view's ``concatenate_to_cache``.
One rank's share of the reference's shard-local path over the ``ATTN_DP`` mesh axis (:278-353) is
``forward_dp_local_shard``; the sum over ranks that follows it there (:355-357) needs more than one GPU.
"""

from __future__ import annotations

from .. import kernels
from ..caching.ragged_page import RaggedPagesMetadata
from ..caching.unified_attention import UnifiedAttentionCacheView
from ._attention_outputs import AttentionOutput
from ._base_operation import OperationImpl, OperationRegistry
from .requirements import CacheType, ExecutionMode, MetadataField, OperationRequirements, RequirementsBuilder


@OperationRegistry.register
class UnifiedAttn(OperationImpl):
    """Causal attention of ragged queries over a paged KV cache with separate K and V pools."""

    @classmethod
    def get_impl_name(cls) -> str | tuple[str]:
        return "unified_attention"

    @classmethod
    def get_requirements(cls, mode: ExecutionMode = ExecutionMode.MIXED) -> OperationRequirements:
        return (RequirementsBuilder("unified_attention")
                .require_metadata(MetadataField.SEQ_LENS | MetadataField.CONTEXT_LENS | MetadataField.POSITIONS
                                  | MetadataField.QUERY_START_LOC | MetadataField.PAGES_TABLES | MetadataField.SLOT_MAPPING)
                .optional_metadata(MetadataField.LOGITS_INDICES)
                .support_cache(CacheType.RAGGED_PAGES)
                .use_cache_view(UnifiedAttentionCacheView)
                .build())

    def forward_native(self, query, cache_view: UnifiedAttentionCacheView | None, cache_metadata: RaggedPagesMetadata,
                       softmax_scale: float | None = None, causal: bool = True, sliding_window: int | None = None,
                       logits_soft_cap: float | None = None, softmax_aux=None, **ignore) -> AttentionOutput:
        if cache_view is None:
            raise ValueError("UnifiedAttn requires `cache_view` (paged KV cache).")
        if not causal:
            raise NotImplementedError("the paged attention kernels are causal-only, as the reference's kernel is")
        is_4d = query.ndim == 4
        shape4 = tuple(query.shape) if is_4d else None
        query_ragged = query.reshape(-1, *query.shape[-2:]).contiguous()
        # The reference passes no live-row count to this kernel (:363-372): every row of context_lens counts and
        # padded rows are those whose query span is empty.
        out = kernels.unified_attention(
            query_ragged, cache_view.key_cache, cache_view.value_cache, cache_metadata.context_lens,
            cache_metadata.pages_tables, cache_metadata.query_start_loc, None, softmax_scale=softmax_scale,
            sliding_window=sliding_window, logits_soft_cap=logits_soft_cap, softmax_aux=softmax_aux)
        if is_4d:
            out = out.reshape(shape4)
        return AttentionOutput(attention_weights=None, attention_outputs=out, cache_view=cache_view)

    def forward_dp_local_shard(self, query, local_key_cache, local_value_cache, cache_metadata: RaggedPagesMetadata,
                               shard_index: int, num_shards: int, softmax_scale: float | None = None,
                               sliding_window: int | None = None, logits_soft_cap: float | None = None, softmax_aux=None,
                               **ignore):
        """What one data-parallel rank computes when the K and V pools are sharded over ranks and every sequence's pages
        live on the rank of its metadata row (the body of the reference's ``shard_map`` at :296-353, before the sum over
        ranks): its rows of the lengths, page tables and ``query_start_loc``, page ids rebased by
        ``shard_index * local_pages``.  The reference also rotates the packed tokens so that the rank's span starts at
        index 0 (its kernel needs ``query_start_loc[0] == 0``, :319-327) and zeroes the other ranks' tokens afterwards
        (:345-353); these kernels take the global token indices as they are and write zeros for tokens outside the
        rank's span, so neither step exists here.  ``query`` is ``[tokens, heads, dim]``; returns the local output."""
        S = int(cache_metadata.context_lens.shape[0])
        if num_shards <= 0 or S % num_shards != 0:
            raise ValueError(f"{S} metadata rows do not divide over {num_shards} shards")
        if not 0 <= shard_index < num_shards:
            raise ValueError(f"shard_index {shard_index} outside [0, {num_shards})")
        rows = S // num_shards
        r0 = shard_index * rows
        local_pages = int(local_key_cache.shape[0])
        tables = cache_metadata.pages_tables.reshape(S, -1)[r0:r0 + rows] - shard_index * local_pages  # ids off the pool are clamped by the kernels
        return kernels.unified_attention(
            query.contiguous(), local_key_cache, local_value_cache, cache_metadata.context_lens[r0:r0 + rows].contiguous(),
            tables.to(cache_metadata.pages_tables.dtype).contiguous(), cache_metadata.query_start_loc[r0:r0 + rows + 1].contiguous(), None,
            softmax_scale=softmax_scale, sliding_window=sliding_window, logits_soft_cap=logits_soft_cap, softmax_aux=softmax_aux)

    def forward_gpu(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)

    def forward_rocm(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)
