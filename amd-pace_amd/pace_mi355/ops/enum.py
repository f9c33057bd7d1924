"""Operator / backend / dtype enums with the reference's member names
(``pace/ops/enum.py:21-80``) plus the one backend this package adds: ``HIP``."""
from __future__ import annotations

from enum import Enum, auto
from typing import List

import torch


class StrEnum(str, Enum):
    """``enum.StrEnum`` of Python >= 3.11: members are their lower-cased names."""

    def _generate_next_value_(name, start, count, last_values):  # noqa: N805
        return name.lower()

    def __str__(self) -> str:
        return str(self.value)

    __format__ = str.__format__


class OperatorType(StrEnum):
    LINEAR = auto()
    REPEATEDKVLINEAR = auto()
    MHA = auto()
    SOFTMAX = auto()
    RELU = auto()
    GELU = auto()
    SILU = auto()
    TANH = auto()
    LAYERNORM = auto()
    RMSNORM = auto()
    ROTARYEMBEDDING = auto()


class FusedOperatorType(StrEnum):
    FUSEDMLPLINEAR = auto()
    FUSEDLINEARRELU = auto()
    FUSEDLINEARGELU = auto()
    FUSEDLINEARSILU = auto()
    FUSEDLINEARMUL = auto()


class BackendType(StrEnum):
    NATIVE = auto()
    JIT = auto()
    TPP = auto()
    IMBPS = auto()
    HIP = auto()  # hand-written gfx950 kernels; the only backend registered here


class DataType(StrEnum):
    FLOAT32 = auto()
    BFLOAT16 = auto()

    @classmethod
    def from_torch(cls, dtype: torch.dtype) -> "DataType":
        if dtype == torch.float32:
            return cls.FLOAT32
        if dtype == torch.bfloat16:
            return cls.BFLOAT16
        raise ValueError(f"Unsupported dtype: {dtype}")

    def to_torch_dtype(self) -> torch.dtype:
        return torch.float32 if self is DataType.FLOAT32 else torch.bfloat16


# Lookup order when the requested backend has no implementation of an operator
# (reference: ``pace/ops/enum.py:72-80``).  HIP leads, so a model configured for
# any of the reference's CPU backends resolves to the gfx950 kernels.
FALLBACK_BACKEND: List[BackendType] = [
    BackendType.HIP,
    BackendType.NATIVE,
    BackendType.JIT,
    BackendType.TPP,
    BackendType.IMBPS,
]
