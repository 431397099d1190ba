"""``unified_attention`` operation (separate K and V pools) backed by the MI355X HIP kernels.

Drop-in for the reference's ``easydel/operations/kernels/unified_attention.py``: the same class and registry
name (:84, :113), requirements (:117-147), call signature of ``forward_native`` (:149-160), 4-D <-> ragged
reshape (:256-262, :395-396) and ``AttentionOutput`` result.  Where the reference hands the arrays to
``ejkernel.modules.unified_attention`` (:363-388) this module hands device pointers to ``librpa_hip.so``.  The
operation reads the pools only: the step's K/V are written before by the view's ``concatenate_to_cache``.
The reference's shard-local path over the ``ATTN_DP`` mesh axis (:290-361) has no one-GPU counterpart.
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

    def forward_gpu(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)

    def forward_rocm(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)
