"""Operator vocabulary of the LLM layer: which part of a decoder block a backend choice applies to
(reference ``pace/llm/ops.py:36-52``; ``OperatorConfig`` maps these names to backends,
``pace/llm/configs.py:500``)."""
from ..ops import BackendType, DataType, MultiHeadAttention, OperatorType, RotaryEmbedding  # noqa: F401
from ..ops.enum import StrEnum

# Mixed-case member names, as the reference's configurations spell them; values are lower case.
LLMOperatorType = StrEnum(
    "LLMOperatorType",
    [(name, name.lower()) for name in ("QKVProjection", "RoPE", "Attention", "OutProjection", "MLP", "Norm", "LMHead")],
    module=__name__,
)

# The same enum under the name the LLM layer uses.
LLMBackendType = BackendType
