from ._attention_outputs import AttentionOutput
from ._base_operation import BaseOperation, EasyDeLBackends, OperationImpl, OperationMetadata, OperationRegistry
from .multi_latent_ragged_page_attention import MultiLatentRaggedPageAttn, MultiLatentRaggedPageAttnV2
from .ragged_page_attention import RaggedPageAttnV2, RaggedPageAttnV3
from .unified_attention import UnifiedAttn
from .requirements import (
    CacheRequirements,
    CacheType,
    ExecutionMode,
    MetadataField,
    MetadataRequirements,
    OperationRequirements,
    RequirementsBuilder,
)

__all__ = [
    "AttentionOutput", "BaseOperation", "EasyDeLBackends", "OperationImpl", "OperationMetadata", "OperationRegistry",
    "RaggedPageAttnV2", "RaggedPageAttnV3", "UnifiedAttn", "MultiLatentRaggedPageAttn", "MultiLatentRaggedPageAttnV2", "CacheRequirements", "CacheType", "ExecutionMode", "MetadataField",
    "MetadataRequirements", "OperationRequirements", "RequirementsBuilder",
]
