"""Names of operators, backends and data types.

The member names are the reference's (``pace/ops/enum.py:21-80``), because models and
configurations written for it spell them out; ``BackendType.HIP`` is the one addition.  Every
member is a lower-case string equal to its own name, so ``BackendType("hip")`` and
``str(OperatorType.MHA) == "mha"`` work as with ``enum.StrEnum`` of Python >= 3.11.
"""
from __future__ import annotations

from enum import Enum
from typing import List

import torch


class StrEnum(str, Enum):
    """String-valued enum whose members print as their value."""

    def __str__(self) -> str:
        return str(self.value)

    __format__ = str.__format__


def _named(cls_name: str, members: str) -> type:
    """Enum class ``cls_name`` with one member per word of ``members`` (value = the word in lower case)."""
    return StrEnum(cls_name, [(word, word.lower()) for word in members.split()], module=__name__)


# Operators of the reference; only MHA and ROTARYEMBEDDING have an implementation in this package.
OperatorType = _named(
    "OperatorType",
    "LINEAR REPEATEDKVLINEAR MHA SOFTMAX RELU GELU SILU TANH LAYERNORM RMSNORM ROTARYEMBEDDING",
)
FusedOperatorType = _named(
    "FusedOperatorType", "FUSEDMLPLINEAR FUSEDLINEARRELU FUSEDLINEARGELU FUSEDLINEARSILU FUSEDLINEARMUL"
)
# The reference's four CPU backends, then the hand-written gfx950 kernels (the only one registered here).
BackendType = _named("BackendType", "NATIVE JIT TPP IMBPS HIP")


class DataType(StrEnum):
    FLOAT32 = "float32"
    BFLOAT16 = "bfloat16"

    @classmethod
    def from_torch(cls, dtype: torch.dtype) -> "DataType":
        for member, torch_dtype in _TORCH_DTYPES.items():
            if torch_dtype == dtype:
                return member
        raise ValueError(f"Unsupported dtype: {dtype}")

    def to_torch_dtype(self) -> torch.dtype:
        return _TORCH_DTYPES[self]


_TORCH_DTYPES = {DataType.FLOAT32: torch.float32, DataType.BFLOAT16: torch.bfloat16}

# Where the registry looks when the requested backend has no implementation of an operator, in
# order.  The reference lists its CPU backends (``pace/ops/enum.py:72-80``); HIP leads here, so a
# model configured for any of them resolves to the gfx950 kernels.
FALLBACK_BACKEND: List[BackendType] = [BackendType[name] for name in ("HIP", "NATIVE", "JIT", "TPP", "IMBPS")]
