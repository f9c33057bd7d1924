"""The reference's two contiguous cache kinds, kept for interface completeness.

``KVCacheType.DYNAMIC`` and ``KVCacheType.BMC`` (reference
``pace/llm/cache.py:170-400``) hold dense ``[B, H, L, D]`` tensors on whatever
device the states live on and return dense tensors, so they pair with the dense
attention kernel.  They are plain tensor bookkeeping (allocation, ``narrow``
views and device-side copies); the accelerated storage is ``KVCacheType.PAGED``.
"""
from __future__ import annotations

import math
import os
from typing import Optional

import torch

from .cache import KVCacheBase

_TOO_LONG = "Cannot remove more tokens than available in cache."


class DynamicKVCache(KVCacheBase):
    """Grows by concatenation; the first update is kept by reference."""

    def __init__(self, max_seq_length: int):
        self.key: Optional[torch.Tensor] = None
        self.value: Optional[torch.Tensor] = None
        self.seq_len = 0
        self.concat_dim = None

    def update_cache(self, key_states, value_states, concat_dim: int):
        self._pin_concat_dim(concat_dim)
        if self.key is None or self.value is None:
            self.key, self.value = key_states, value_states
        else:
            self.key = torch.cat((self.key, key_states), dim=concat_dim)
            self.value = torch.cat((self.value, value_states), dim=concat_dim)
        self.seq_len = int(self.key.size(concat_dim))
        return self.key, self.value

    def remove_cache(self, remove_len: int) -> None:
        if self.key is None or self.value is None:
            return
        if remove_len > self.seq_len:
            raise ValueError(_TOO_LONG)
        self.seq_len -= remove_len
        self.key = self.key.narrow(self.concat_dim, 0, self.seq_len)
        self.value = self.value.narrow(self.concat_dim, 0, self.seq_len)


class BMCKVCache(KVCacheBase):
    """Zero-padded buffer that is re-made ``tokens_per_split`` rows larger whenever
    an update would fill it; the whole padded buffer is what callers get back, and
    ``update_mask`` pads the additive mask to the same width with ``finfo.min``."""

    def __init__(self, max_seq_length: int):
        n_splits = int(os.getenv("PACE_BMC_NUM_SPLITS", int(math.sqrt(max_seq_length))))
        self.tokens_per_split = max_seq_length // n_splits
        self.key: Optional[torch.Tensor] = None
        self.value: Optional[torch.Tensor] = None
        self.seq_len = 0
        self.concat_dim = None

    def _padded(self, n_tokens: int) -> int:
        step = self.tokens_per_split
        return ((n_tokens - 1) // step + 1) * step

    def update_mask(self, attn_mask: torch.Tensor, input_size: int) -> torch.Tensor:
        pad = self._padded(input_size) - input_size
        tail = attn_mask.new_full(attn_mask.shape[:-1] + (pad,), torch.finfo(attn_mask.dtype).min)
        return torch.cat((attn_mask, tail), dim=-1)

    def remove_cache(self, remove_len: int) -> None:
        if self.key is None or self.value is None:
            return
        if remove_len > self.seq_len:
            raise ValueError(_TOO_LONG)
        self.seq_len -= remove_len

    def update_cache(self, key_states, value_states, concat_dim: int):
        self._pin_concat_dim(concat_dim)
        ax = self.concat_dim
        end = self.seq_len + key_states.size(ax)
        if self.key is None or self.value is None or end >= self.key.size(ax):
            shape = list(key_states.shape)
            shape[ax] = self._padded(end)
            fresh = [key_states.new_zeros(shape), key_states.new_zeros(shape)]
            for new, old in zip(fresh, (self.key, self.value)):
                if self.key is not None and self.value is not None:
                    new.narrow(ax, 0, old.size(ax)).copy_(old)
            self.key, self.value = fresh
        self.key.narrow(ax, self.seq_len, key_states.size(concat_dim)).copy_(key_states)
        self.value.narrow(ax, self.seq_len, value_states.size(concat_dim)).copy_(value_states)
        self.seq_len = end
        return self.key, self.value
