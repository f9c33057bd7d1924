"""``MultiHeadAttention`` operator (reference: ``pace/ops/attention.py:15-41``)."""
from __future__ import annotations

from typing import Optional

import torch

from .base import OperatorBase
from .enum import BackendType, DataType, OperatorType


class MultiHeadAttention(OperatorBase):
    """``softmax(Q K^T / sqrt(D) + mask) V``.

    ``key`` / ``value`` are either dense ``[B, H, L, D]`` tensors, as in the
    reference, or the paged views a ``PagedKVCache.update_cache`` returns.
    """

    @property
    def operator_type(self):
        return OperatorType.MHA

    def __init__(self, dtype: Optional[DataType] = None, backend_impl: BackendType = BackendType.NATIVE):
        self.dtype = dtype
        super().__init__(backend_impl=backend_impl, dtype=dtype)

    def forward(self, query, key, value, attention_mask: Optional[torch.Tensor] = None):
        return self.backend.execute(query=query, key=key, value=value, attention_mask=attention_mask)

    def extra_repr(self) -> str:
        return f"dtype={self.dtype}, backend={self.backend}"
