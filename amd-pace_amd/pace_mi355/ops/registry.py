"""Backend registry: ``(operator, backend, dtype) -> implementation class``.

Same contract as ``pace/ops/registry.py:20-106`` of the reference: decorator
registration, duplicate registration asserts, exact match first, then the
``FALLBACK_BACKEND`` order for plain operators (never for fused ones), and an
assertion when nothing matches.
"""
from __future__ import annotations

from collections import defaultdict
from typing import Dict, List, Tuple, Type, Union

from ..utils.logging import PACE_ASSERT, PACE_DEBUG
from .enum import BackendType, DataType, FALLBACK_BACKEND, FusedOperatorType, OperatorType

AnyOperator = Union[OperatorType, FusedOperatorType]


class BackendRegistry:
    def __init__(self) -> None:
        self._registry: Dict[AnyOperator, Dict[Tuple[BackendType, DataType], Type]] = defaultdict(dict)

    def register(self, operator: AnyOperator, backend: BackendType, dtype: List[DataType]):
        taken = self._registry.get(operator, {})
        for dt in dtype:
            if (backend, dt) in taken:
                PACE_ASSERT(False, f"Duplicate registration of {operator} with backend {backend} and dtype {dt}")

        def decorator(cls):
            for dt in dtype:
                self._registry[operator][(backend, dt)] = cls
            return cls

        return decorator

    def get_available_backends(self, operator: AnyOperator) -> List[Tuple[BackendType, DataType]]:
        PACE_DEBUG(f"Getting available backends for {operator}")
        if operator not in self._registry:
            PACE_DEBUG(f"Operator {operator} not registered, returning empty list")
            return []
        return list(self._registry[operator].keys())

    def get(self, operator: AnyOperator, backend: BackendType, dtype: DataType):
        PACE_DEBUG(f"Getting backend for {operator}, {backend}, {dtype}")
        if operator not in self._registry:
            PACE_DEBUG(
                f"Operator {operator} not registered, this operator might be a new one, or one without a backend"
            )
            return None
        impls = self._registry[operator]
        if (backend, dtype) in impls:
            PACE_DEBUG(f"Found backend {backend} for {operator} with {dtype}")
            return impls[(backend, dtype)]
        if isinstance(operator, FusedOperatorType):
            PACE_DEBUG(
                f"Fused operator {operator} with backend {backend} and dtype {dtype} not found in registry."
                "It will be handled by the default forward method."
            )
            return None
        PACE_DEBUG(f"Backend {backend} not found for {operator} with {dtype}. Trying fallback backends...")
        for candidate in FALLBACK_BACKEND:
            if (candidate, dtype) in impls:
                PACE_DEBUG(f"Using fallback backend {candidate} for {operator} with {dtype}")
                return impls[(candidate, dtype)]
        PACE_ASSERT(False, f"No backend found for {operator} with {backend}, {dtype}")

    def __repr__(self) -> str:
        return str(self._registry)


backend_registry = BackendRegistry()
