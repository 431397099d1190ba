"""Declarations an operation makes about the metadata and cache it needs.

Same names and meaning as the reference's ``easydel/operations/requirements`` package
(``types.py:26-153``, ``requirements.py:27-240``, ``builder.py:30-176``): the engine asks an operation
which metadata fields to build and which cache view class to allocate.
"""

from __future__ import annotations

from dataclasses import dataclass, field, replace
from enum import Enum, Flag, auto


class ExecutionMode(Enum):
    PREFILL = "prefill"
    DECODE = "decode"
    MIXED = "mixed"


class MetadataField(Flag):
    NONE = 0
    SEQ_LENS = auto()
    CONTEXT_LENS = auto()
    POSITIONS = auto()
    QUERY_START_LOC = auto()
    PAGES_TABLES = auto()
    SLOT_MAPPING = auto()
    REQUEST_DISTRIBUTION = auto()
    HAS_INITIAL_STATE = auto()
    STATE_INDICES = auto()
    LOGITS_INDICES = auto()

    @classmethod
    def basic(cls) -> "MetadataField":
        return cls.SEQ_LENS | cls.POSITIONS

    @classmethod
    def ragged(cls) -> "MetadataField":
        return cls.basic() | cls.CONTEXT_LENS | cls.QUERY_START_LOC | cls.PAGES_TABLES

    @classmethod
    def paged_v2(cls) -> "MetadataField":
        return cls.ragged() | cls.SLOT_MAPPING

    @classmethod
    def paged_v3(cls) -> "MetadataField":
        return cls.ragged() | cls.REQUEST_DISTRIBUTION


class CacheType(Flag):
    NONE = 0
    TRANSFORMER = auto()
    RAGGED_PAGES = auto()
    RECURRENT = auto()
    HYBRID = auto()

    @classmethod
    def any(cls) -> "CacheType":
        return cls.TRANSFORMER | cls.RAGGED_PAGES | cls.RECURRENT | cls.HYBRID

    def is_compatible_with(self, other: "CacheType") -> bool:
        return bool(self & other)


@dataclass(frozen=True)
class MetadataRequirements:
    required: MetadataField = MetadataField.NONE
    optional: MetadataField = MetadataField.NONE

    @property
    def all_fields(self) -> MetadataField:
        return self.required | self.optional

    def is_satisfied_by(self, available: MetadataField) -> bool:
        return (self.required & available) == self.required

    def missing_fields(self, available: MetadataField) -> MetadataField:
        return self.required & ~available


@dataclass(frozen=True)
class CacheRequirements:
    supported: CacheType = CacheType.NONE
    preferred: CacheType | None = None
    requires_cache: bool = True
    cache_view_class: type | None = None

    def is_compatible_with(self, cache_type: CacheType) -> bool:
        return bool(self.supported & cache_type)


@dataclass(frozen=True)
class OperationRequirements:
    name: str = ""
    metadata: MetadataRequirements = field(default_factory=MetadataRequirements)
    cache: CacheRequirements = field(default_factory=CacheRequirements)

    @classmethod
    def create(cls, name="", required_metadata=MetadataField.NONE, optional_metadata=MetadataField.NONE,
               supported_cache=CacheType.NONE, preferred_cache=None, requires_cache=True, cache_view_class=None):
        return cls(name, MetadataRequirements(required_metadata, optional_metadata),
                   CacheRequirements(supported_cache, preferred_cache, requires_cache, cache_view_class))

    def with_requires_cache(self, requires_cache: bool) -> "OperationRequirements":
        return replace(self, cache=replace(self.cache, requires_cache=requires_cache,
                                           cache_view_class=self.cache.cache_view_class if requires_cache else None))


class RequirementsBuilder:
    """Fluent builder: ``RequirementsBuilder(name).require_metadata(...).support_cache(...).build()``."""

    def __init__(self, name: str = ""):
        self._name = name
        self._required = MetadataField.NONE
        self._optional = MetadataField.NONE
        self._supported = CacheType.NONE
        self._preferred = None
        self._requires_cache = True
        self._cache_view_class = None

    def require_metadata(self, fields: MetadataField) -> "RequirementsBuilder":
        self._required |= fields
        return self

    def optional_metadata(self, fields: MetadataField) -> "RequirementsBuilder":
        self._optional |= fields
        return self

    def support_cache(self, cache_types: CacheType) -> "RequirementsBuilder":
        self._supported = cache_types
        return self

    def add_cache_support(self, cache_types: CacheType) -> "RequirementsBuilder":
        self._supported |= cache_types
        return self

    def prefer_cache(self, cache_type: CacheType) -> "RequirementsBuilder":
        self._preferred = cache_type
        return self

    def requires_cache(self, value: bool = True) -> "RequirementsBuilder":
        self._requires_cache = value
        return self

    def no_cache_required(self) -> "RequirementsBuilder":
        return self.requires_cache(False)

    def use_cache_view(self, cache_view_class: type) -> "RequirementsBuilder":
        self._cache_view_class = cache_view_class
        return self

    def build(self) -> OperationRequirements:
        return OperationRequirements.create(self._name, self._required, self._optional, self._supported, self._preferred,
                                            self._requires_cache, self._cache_view_class)
