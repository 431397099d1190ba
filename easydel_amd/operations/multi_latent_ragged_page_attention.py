"""``multi_latent_ragged_page_attention_v1`` / ``_v2`` operations backed by the MI355X HIP kernels.

Drop-in for the reference's ``easydel/operations/kernels/multi_latent_ragged_page_attention.py``: the same two
classes and registry names (:262, :283, :800, :812), requirements (:763-796), keyword signature (:285-301), tensor
normalisation and error messages (:123-180, :340-378), and ``AttentionOutput`` result with the updated view (:636-637).
Where the reference hands the arrays to ``ejkernel.modules.multi_latent_ragged_page_attention`` (:495-511, :611-624;
v2 :1019-1030, :1090-1101) this module hands device pointers to ``librpa_hip.so``.  The two versions differ in the
reference only by the block-size hints they pass to ejkernel; here they are one implementation.  The shard-local path
over the ``ATTN_DP`` mesh axis (:437-560) has no one-GPU counterpart.
"""

from __future__ import annotations

import logging

import torch

from .. import kernels
from ..caching.mla_ragged_page import MLARaggedPagesCacheView
from ._attention_outputs import AttentionOutput
from ._base_operation import OperationImpl, OperationRegistry
from .requirements import CacheType, ExecutionMode, MetadataField, OperationRequirements, RequirementsBuilder

logger = logging.getLogger(__name__)


def _reshape_query_tensor(x, name: str):
    """Rank-4 ``[batch, seq, heads, dim]`` -> ``[tokens, heads, dim]``; rank-3 unchanged (reference :123-144)."""
    if x is None:
        return None
    if x.ndim == 4:
        return x.reshape(-1, x.shape[-2], x.shape[-1])
    if x.ndim == 3:
        return x
    raise ValueError(f"`{name}` must be rank-3 or rank-4, got rank-{x.ndim}.")


def _reshape_feature_tensor(x, name: str):
    """Rank-4 -> ``[tokens, heads, dim]``, rank-3 ``[batch, seq, dim]`` -> ``[tokens, dim]``, rank-2 unchanged (:147-180)."""
    if x is None:
        return None
    if x.ndim == 4:
        return x.reshape(-1, x.shape[-2], x.shape[-1])
    if x.ndim == 3:
        return x.reshape(-1, x.shape[-1])
    if x.ndim == 2:
        return x
    raise ValueError(f"`{name}` must be rank-2, rank-3, or rank-4, got rank-{x.ndim}.")


def _resolve_distribution(cache_metadata) -> torch.Tensor:
    """``[decode_end, prefill_end, total]`` of the batch, computed on the device from the metadata when it carries
    none (reference :225-258; no host round trip, as there)."""
    dist = getattr(cache_metadata, "request_distribution", None)
    if dist is not None:
        return dist.to(torch.int32)
    qsl, ctx = cache_metadata.query_start_loc, cache_metadata.context_lens
    scheduled = qsl[1:] - qsl[:-1]
    has_tokens = scheduled > 0
    is_decode = (scheduled == 1) & (ctx > 1) & has_tokens
    decode = is_decode.sum()
    return torch.stack([decode, decode + (has_tokens & ~is_decode).sum(), has_tokens.sum()]).to(torch.int32)


class _MultiLatentRaggedPageAttn(OperationImpl):
    _NAME = ""

    @classmethod
    def get_impl_name(cls) -> str | tuple[str]:
        return cls._NAME

    @classmethod
    def get_requirements(cls, mode: ExecutionMode = ExecutionMode.MIXED) -> OperationRequirements:
        del mode
        return (RequirementsBuilder("multi_latent_ragged_page_attention")
                .require_metadata(MetadataField.SEQ_LENS | MetadataField.CONTEXT_LENS | MetadataField.POSITIONS
                                  | MetadataField.QUERY_START_LOC | MetadataField.PAGES_TABLES
                                  | MetadataField.REQUEST_DISTRIBUTION)
                .optional_metadata(MetadataField.LOGITS_INDICES)
                .support_cache(CacheType.RAGGED_PAGES)
                .use_cache_view(MLARaggedPagesCacheView)
                .build())

    def forward_core(self, queries_nope, queries_pe, keys_values, keys_pe, cache_view, cache_metadata,
                     softmax_scale: float | None = None, logits_soft_cap: float | None = None,
                     sliding_window: int | None = None, vmem_limit_bytes: int | None = None,
                     mask_value: float | None = None, q_scale: float | None = None, k_scale: float | None = None,
                     v_scale: float | None = None, softmax_aux=None, **ignore) -> AttentionOutput:
        name = self.get_impl_name()
        if keys_pe is None:
            raise ValueError(f"{name} requires `keys_pe`. Pass it as `keys_pe=` (or `k_pe=`).")
        if q_scale is not None or k_scale is not None or v_scale is not None:
            raise NotImplementedError(f"{name}: q_scale / k_scale / v_scale (quantised operands) are not supported")
        is_4d = queries_nope.ndim == 4
        shape4 = tuple(queries_nope.shape) if is_4d else None
        queries_nope = _reshape_query_tensor(queries_nope, "queries_nope")
        queries_pe = _reshape_query_tensor(queries_pe, "queries_pe")
        keys_values = _reshape_feature_tensor(keys_values, "keys_values")
        keys_pe = _reshape_feature_tensor(keys_pe, "keys_pe")
        if queries_nope.shape[:2] != queries_pe.shape[:2]:
            raise ValueError("`queries_nope` and `queries_pe` must share [total_tokens, num_q_heads]. "
                             f"Got {tuple(queries_nope.shape[:2])} vs {tuple(queries_pe.shape[:2])}.")
        if keys_values.ndim not in (2, 3):
            raise ValueError("`keys_values` must be rank-2 [total_tokens, kv_lora_rank] or "
                             f"rank-3 [total_tokens, num_kv_heads, kv_lora_rank]. Got shape={tuple(keys_values.shape)}.")
        if keys_values.ndim == 3:
            raise NotImplementedError(f"{name}: per-head `keys_values` [tokens, heads, rank] are not supported; "
                                      "the latent cache holds one row per token")
        if keys_pe.ndim != 2:
            raise ValueError(f"`keys_pe` must be rank-2 [total_tokens, qk_pe_dim]. Got shape={tuple(keys_pe.shape)}.")
        if keys_values.shape[0] != queries_nope.shape[0]:
            raise ValueError("`keys_values` token dimension must match `queries_nope` token dimension. "
                             f"Got keys_values={keys_values.shape[0]} vs queries_nope={queries_nope.shape[0]}. "
                             "Pass explicit MLA tensors (`keys_values`, `keys_pe`) instead of standard value heads.")
        if keys_pe.shape[0] != queries_nope.shape[0]:
            raise ValueError("`keys_pe` token dimension must match `queries_nope` token dimension. "
                             f"Got keys_pe={keys_pe.shape[0]} vs queries_nope={queries_nope.shape[0]}.")
        kv_pages = cache_view.kv_pages
        if keys_values.dtype != kv_pages.dtype or keys_pe.dtype != kv_pages.dtype:
            if kv_pages.element_size() < max(keys_values.element_size(), keys_pe.element_size()):
                logger.warning("Casting keys_values/keys_pe from %s to lower-precision KV cache dtype %s; "
                               "this may reduce numerical fidelity.", keys_values.dtype, kv_pages.dtype)
            keys_values = keys_values.to(kv_pages.dtype)
            keys_pe = keys_pe.to(kv_pages.dtype)
        distribution = _resolve_distribution(cache_metadata)
        # the reference hands the kernel [0, 0, total] (:376-378): the first two entries are scheduling hints only
        distribution = torch.stack([torch.zeros_like(distribution[2]), torch.zeros_like(distribution[2]), distribution[2]])
        output, kv_pages = kernels.mla_ragged_paged_attention(
            queries_nope.contiguous(), queries_pe.to(queries_nope.dtype).contiguous(), keys_values.contiguous(),
            keys_pe.contiguous(), kv_pages, cache_metadata.context_lens, cache_metadata.pages_tables.reshape(-1),
            cache_metadata.query_start_loc, distribution.contiguous(), softmax_scale=softmax_scale,
            sliding_window=sliding_window, logits_soft_cap=logits_soft_cap, softmax_aux=softmax_aux)
        cache_view.kv_pages = kv_pages
        if is_4d:
            output = output.reshape(shape4)
        return AttentionOutput(attention_weights=None, attention_outputs=output, cache_view=cache_view)

    def forward_core_dp_local_shard(self, queries_nope, queries_pe, keys_values, keys_pe, local_kv_pages, cache_metadata,
                                    shard_index: int, num_shards: int, softmax_scale: float | None = None,
                                    logits_soft_cap: float | None = None, sliding_window: int | None = None,
                                    softmax_aux=None, **ignore):
        """One data-parallel rank's share when the latent pages are sharded over ranks and every sequence's pages live
        on the rank of its metadata row (the body of the reference's ``shard_map`` at :507-566, before the sum over
        ranks): metadata rows sliced, page ids rebased and clipped, distribution recomputed, fused write + attention on
        the rank's pages; the rows of other ranks' tokens come back as zeros.  Operands already flattened
        (``[tokens, heads, dim]`` / ``[tokens, dim]``) and in the page dtype.  Returns ``(local_output, local_kv_pages)``;
        the ranks' outputs are summed in float32 (``ragged_page_attention.dp_local_reduce``)."""
        from .ragged_page_attention import dp_local_metadata

        context_lens, tables, query_start_loc, distribution = dp_local_metadata(cache_metadata, shard_index, num_shards,
                                                                                int(local_kv_pages.shape[0]))
        distribution = torch.stack([torch.zeros_like(distribution[2]), torch.zeros_like(distribution[2]), distribution[2]])
        return kernels.mla_ragged_paged_attention(
            queries_nope.contiguous(), queries_pe.to(queries_nope.dtype).contiguous(), keys_values.to(local_kv_pages.dtype).contiguous(),
            keys_pe.to(local_kv_pages.dtype).contiguous(), local_kv_pages, context_lens, tables, query_start_loc,
            distribution.contiguous(), softmax_scale=softmax_scale, sliding_window=sliding_window,
            logits_soft_cap=logits_soft_cap, softmax_aux=softmax_aux)

    def forward_native(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_core(*args, **kwargs)

    def forward_gpu(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)

    def forward_rocm(self, *args, **kwargs) -> AttentionOutput:
        return self.forward_native(*args, **kwargs)


@OperationRegistry.register
class MultiLatentRaggedPageAttn(_MultiLatentRaggedPageAttn):
    """MLA over latent ragged pages, version 1 of the reference's two registrations."""

    _NAME = "multi_latent_ragged_page_attention_v1"


@OperationRegistry.register
class MultiLatentRaggedPageAttnV2(_MultiLatentRaggedPageAttn):
    """MLA over latent ragged pages, version 2 (the serving engine's default, esurge_engine.py:114)."""

    _NAME = "multi_latent_ragged_page_attention_v2"
