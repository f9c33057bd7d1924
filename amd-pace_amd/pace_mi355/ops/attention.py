"""The attention operator models instantiate (reference: ``pace/ops/attention.py:15-41``).

``MultiHeadAttention(dtype, backend_impl)(query, key, value, attention_mask)`` computes
``softmax(Q K^T / sqrt(D) + mask) V`` through whichever backend the registry resolves; in this
package that is always the gfx950 one (``backends/hip.py``), whatever name was asked for.

Shapes: ``query [B, Hq, S, D]``; ``key`` / ``value`` either dense ``[B, Hq, L, D]`` tensors, as in the
reference, or the paged views ``PagedKVCache.update_cache`` returns (then GQA is resolved inside
the kernel and nothing is expanded); ``attention_mask`` additive, broadcastable ``[B|1, 1|Hq, S|1, L]``.
"""
from __future__ import annotations

from typing import Optional

import torch

from .base import OperatorBase
from .enum import BackendType, DataType, OperatorType


class MultiHeadAttention(OperatorBase):
    operator_type = OperatorType.MHA

    def __init__(self, dtype: Optional[DataType] = None, backend_impl: BackendType = BackendType.NATIVE):
        # OperatorBase turns ``dtype`` into a DataType member and resolves the backend class.
        super().__init__(backend_impl=backend_impl, dtype=dtype)

    def forward(self, query, key, value, attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.backend is None:  # nothing registered for this dtype: there is no eager fallback to hide behind
            raise RuntimeError(f"no attention backend registered for {self.dtype}")
        return self.backend.execute(query=query, key=key, value=value, attention_mask=attention_mask)

    def extra_repr(self) -> str:
        return f"dtype={self.dtype}, backend={self.backend}"
