"""Which class implements an operator for a backend and a data type.

Behaviour follows ``pace/ops/registry.py:20-106`` of the reference, including the three messages
its tests look for: registration through a decorator, an assertion on a second registration of the
same (operator, backend, dtype), lookup by exact match first and then along ``FALLBACK_BACKEND``
(plain operators only; a fused operator without an exact match is left to its default forward), an
assertion when a registered operator has nothing for the request, ``None`` for an operator nobody
registered.
"""
from __future__ import annotations

from typing import Dict, Iterable, Iterator, List, Optional, Tuple, Type, Union

from ..utils.logging import PACE_ASSERT, PACE_DEBUG
from . import enum as _names
from .enum import BackendType, DataType, FusedOperatorType, OperatorType

# Kept as a module attribute as well: callers (and tests) may edit the list in place.
FALLBACK_BACKEND = _names.FALLBACK_BACKEND

AnyOperator = Union[OperatorType, FusedOperatorType]
Slot = Tuple[BackendType, DataType]


class BackendRegistry:
    def __init__(self) -> None:
        self._table: Dict[AnyOperator, Dict[Slot, Type]] = {}

    # -- registration -------------------------------------------------------------------------
    def register(self, operator: AnyOperator, backend: BackendType, dtype: Iterable[DataType]):
        """Class decorator: ``@backend_registry.register(OperatorType.MHA, BackendType.HIP, [DataType.BFLOAT16])``."""
        dtypes = list(dtype)
        taken = self._table.get(operator, {})
        for dt in (d for d in dtypes if (backend, d) in taken):
            PACE_ASSERT(False, f"Duplicate registration of {operator} with backend {backend} and dtype {dt}")

        def bind(implementation: Type) -> Type:
            slots = self._table.setdefault(operator, {})
            slots.update({(backend, dt): implementation for dt in dtypes})
            return implementation

        return bind

    # -- lookup -------------------------------------------------------------------------------
    def get_available_backends(self, operator: AnyOperator) -> List[Slot]:
        slots = self._table.get(operator)
        PACE_DEBUG(f"{operator}: {len(slots) if slots else 0} (backend, dtype) slots registered")
        return list(slots) if slots else []

    def _candidates(self, operator: AnyOperator, backend: BackendType) -> Iterator[BackendType]:
        yield backend
        if not isinstance(operator, FusedOperatorType):
            yield from FALLBACK_BACKEND

    def get(self, operator: AnyOperator, backend: BackendType, dtype: DataType) -> Optional[Type]:
        slots = self._table.get(operator)
        if slots is None:
            PACE_DEBUG(f"Operator {operator} not registered, this operator might be a new one, or one without a backend")
            return None
        for rank, candidate in enumerate(self._candidates(operator, backend)):
            implementation = slots.get((candidate, dtype))
            if implementation is not None:
                PACE_DEBUG(f"{operator}/{dtype}: {'requested' if rank == 0 else 'fallback'} backend {candidate} -> {implementation.__name__}")
                return implementation
        if isinstance(operator, FusedOperatorType):
            PACE_DEBUG(
                f"Fused operator {operator} with backend {backend} and dtype {dtype} not found in registry."
                "It will be handled by the default forward method."
            )
            return None
        PACE_ASSERT(False, f"No backend found for {operator} with {backend}, {dtype}")
        return None

    def __repr__(self) -> str:
        return repr(self._table)


backend_registry = BackendRegistry()
