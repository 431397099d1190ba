"""Operation base class and registry: the plug-in interface attention layers select kernels through.

Mirrors ``easydel/operations/_base_operation.py`` of the reference: ``BaseOperation.__call__`` dispatches
on the metadata's backend (:253-288), ``OperationRegistry.register`` files a class under the name(s) its
``get_impl_name()`` returns and overwrites an existing entry with a warning (:310-350), ``get`` raises
``ValueError`` for unknown names (:352-374), ``create`` instantiates with the metadata (:376-410).
"""

from __future__ import annotations

import logging
import os
import typing as tp
from abc import ABC, abstractmethod
from dataclasses import dataclass, field
from enum import Enum

from .requirements import CacheType, ExecutionMode, MetadataField, OperationRequirements

logger = logging.getLogger(__name__)


class EasyDeLBackends(str, Enum):
    CPU = "cpu"
    GPU = "gpu"
    TPU = "tpu"
    TT = "tt"


def check_bool_flag(name: str, default: bool = False) -> bool:
    """Environment flag parsing as the reference's ``utils/helpers.py:437-458`` does it."""
    val = os.environ.get(name)
    if val is None:
        return default
    return val.strip().lower() in ("1", "true", "yes", "y", "on", "t")


@dataclass
class OperationMetadata:
    """The slice of the reference's ``OperationMetadata`` (``_operation_meta.py:87-376``) this path reads:
    runtime dtype, softmax scale, backend, per-operation tuning configs."""

    runtime_dtype: tp.Any = None
    runtime_softmax_dtype: tp.Any = None
    softmax_scale: float | None = None
    soft_cap: float | None = None
    backend: EasyDeLBackends = EasyDeLBackends.GPU
    platform: str = "rocm"
    requires_cache: bool = True
    operation_configs: dict = field(default_factory=dict)
    mesh: tp.Any = None
    partition_manager: tp.Any = None

    def get_operation_config(self, impl_name: str):
        return (self.operation_configs or {}).get(impl_name)


class BaseOperation(ABC):
    metadata: OperationMetadata | None = None

    @classmethod
    @abstractmethod
    def get_impl_name(cls) -> str | tuple[str, ...]:
        """Name(s) the registry files this implementation under."""

    @abstractmethod
    def get_impl_metadata(self) -> OperationMetadata:
        """The metadata passed at construction."""

    @classmethod
    def get_requirements(cls, mode: ExecutionMode = ExecutionMode.MIXED) -> OperationRequirements:
        name = cls.get_impl_name()
        if isinstance(name, tuple):
            name = name[0]
        return OperationRequirements.create(name=name, required_metadata=MetadataField.basic(), supported_cache=CacheType.any())

    @abstractmethod
    def forward_native(self, *args, **kwargs) -> tp.Any:
        """Backend-agnostic implementation; every subclass provides it."""

    def forward_gpu(self, *args, **kwargs):
        return self.forward_native(*args, **kwargs)

    def forward_rocm(self, *args, **kwargs):
        return self.forward_gpu(*args, **kwargs)

    def forward_cuda(self, *args, **kwargs):
        return self.forward_gpu(*args, **kwargs)

    def forward_tpu(self, *args, **kwargs):
        return self.forward_native(*args, **kwargs)

    def forward_tt(self, *args, **kwargs):
        return self.forward_native(*args, **kwargs)

    def forward_cpu(self, *args, **kwargs):
        return self.forward_native(*args, **kwargs)

    def __call__(self, *args, **kwargs):
        if check_bool_flag("FORCE_NATIVE_RUNTIME", False):
            return self.forward_native(*args, **kwargs)
        backend = self.metadata.backend
        backend = getattr(backend, "value", backend)
        if backend == "tpu":
            return self.forward_tpu(*args, **kwargs)
        if backend == "gpu":
            return self.forward_gpu(*args, **kwargs)
        if backend == "tt":
            return self.forward_tt(*args, **kwargs)
        if backend == "cpu":
            return self.forward_native(*args, **kwargs)
        raise RuntimeError(f"unknown backend at OperationImpl! {self.metadata.backend}")


class OperationImpl(BaseOperation):
    """Concrete base holding the metadata (reference ``_operation_impl.py:96-131``)."""

    def __init__(self, metadata: OperationMetadata | None = None):
        self.metadata = metadata if metadata is not None else OperationMetadata()

    def get_impl_metadata(self) -> OperationMetadata:
        return self.metadata


class OperationRegistry:
    _registry: tp.ClassVar[dict[str, type[BaseOperation]]] = {}

    @classmethod
    def register(cls, impl_cls):
        names = impl_cls.get_impl_name()
        if not isinstance(names, (list, tuple)):
            names = [names]
        for name in names:
            if name in cls._registry:
                logger.warning(f"Operation implementation '{name}' already registered. Overwriting.")
            cls._registry[name] = impl_cls
        return impl_cls

    @classmethod
    def get(cls, impl_name: str) -> type[BaseOperation]:
        if impl_name not in cls._registry:
            raise ValueError(
                f"Operation implementation '{impl_name}' not found. Available implementations: {list(cls._registry.keys())}")
        return cls._registry[impl_name]

    @classmethod
    def create(cls, impl_name: str, metadata: OperationMetadata, requires_cache: bool | None = None) -> BaseOperation:
        if requires_cache is not None:
            metadata.requires_cache = requires_cache
        return cls.get(impl_name)(metadata)

    @classmethod
    def list_implementations(cls) -> list[str]:
        return list(cls._registry.keys())
