"""LLM-level operator names (reference ``pace/llm/ops.py:36-52``)."""
from enum import auto

from ..ops import BackendType, DataType, MultiHeadAttention, OperatorType  # noqa: F401
from ..ops.enum import StrEnum


class LLMOperatorType(StrEnum):
    QKVProjection = auto()
    RoPE = auto()
    Attention = auto()
    OutProjection = auto()
    MLP = auto()
    Norm = auto()
    LMHead = auto()


LLMBackendType = BackendType
