"""The gfx950 implementation of ``OperatorType.MHA``.

Registered the way the reference registers its backends
(``pace/ops/backends/jit.py:31-47``).  Dense ``[B, H, L, D]`` keys / values go
through ``torch.ops.pace.attention``; the paged views a ``PagedKVCache`` returns
go to the paged kernels, which read the block pool in place.
"""
from __future__ import annotations

from typing import Optional

import torch

from ..base import BackendBase
from ..enum import BackendType, DataType, OperatorType
from ..registry import backend_registry


@backend_registry.register(OperatorType.MHA, BackendType.HIP, [DataType.FLOAT32, DataType.BFLOAT16])
class HIPAttention(BackendBase):
    def execute(self, query: torch.Tensor, key, value, attention_mask: Optional[torch.Tensor] = None) -> torch.Tensor:
        from ...llm.cache import PagedKVView

        if isinstance(key, PagedKVView):
            if not isinstance(value, PagedKVView) or value.cache is not key.cache:
                raise RuntimeError("key and value must be the two views of one PagedKVCache")
            return key.cache.attend(query, attention_mask)
        query, key, value = query.contiguous(), key.contiguous(), value.contiguous()
        if attention_mask is None:
            # The op dereferences its mask (csrc/ops/attention.cpp:26-29 of the
            # reference); an absent mask is the all-zero one.
            attention_mask = query.new_zeros((1, 1, 1, key.size(2)))
        return torch.ops.pace.attention(query, key, value, attention_mask, False)
