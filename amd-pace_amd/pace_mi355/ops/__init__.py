from .enum import BackendType, DataType, FusedOperatorType, OperatorType  # noqa: F401
from .registry import backend_registry  # noqa: F401
from .base import BackendBase, OperatorBase  # noqa: F401
from .attention import MultiHeadAttention  # noqa: F401
from .rotary_embedding import RotaryEmbedding  # noqa: F401
from . import backends  # noqa: F401  (registers the implementations)
from . import torch_op  # noqa: F401  (defines torch.ops.pace.attention)

__all__ = ["OperatorType", "FusedOperatorType", "BackendType", "DataType", "MultiHeadAttention", "RotaryEmbedding",
           "backend_registry"]
