"""Operator / backend base classes (reference: ``pace/ops/base.py:17-113``)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Optional, Type

from torch import get_default_dtype, nn

from .enum import BackendType, DataType, OperatorType
from .registry import backend_registry


class BackendBase(ABC):
    """One implementation of one operator; ``execute`` does the work."""

    def create_extra_params(self, layer: nn.Module) -> None:
        """Hook run once from the operator's constructor."""

    def preprocess(self, layer: nn.Module) -> None:
        """Optional hook after weights are loaded."""

    @abstractmethod
    def execute(self, *args, **kwargs):
        ...

    def __repr__(self) -> str:
        return type(self).__name__


class OperatorBase(nn.Module, ABC):
    """Resolves its backend class through the registry at construction."""

    def __init__(self, backend_impl: Optional[BackendType] = None, dtype: Optional[DataType] = None):
        super().__init__()
        if dtype is None:
            dtype = get_default_dtype()
        if not isinstance(dtype, DataType):
            dtype = DataType.from_torch(dtype)
        self.dtype = dtype
        self.backend_impl = backend_impl
        self.backend_cls: Optional[Type[BackendBase]] = backend_registry.get(self.operator_type, backend_impl, dtype)
        self.backend: Optional[BackendBase] = None
        if self.backend_cls is not None:
            self.backend = self.backend_cls()
            self.backend.create_extra_params(self)

    @property
    @abstractmethod
    def operator_type(self) -> OperatorType:
        ...

    def load_weights(self, *args, **kwargs) -> None:
        """Operators with parameters override this."""

    @abstractmethod
    def forward(self, *args, **kwargs):
        ...

    @abstractmethod
    def extra_repr(self) -> str:
        ...
