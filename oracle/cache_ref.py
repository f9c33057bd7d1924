"""Oracle: the reference's two contiguous KV caches, restated on CPU tensors.

TEST INFRASTRUCTURE -- see ``oracle/__init__.py``.  Follows
``pace/llm/cache.py`` of the reference (line numbers cited per function).
The tensors are whatever the caller hands in (the reference models hand in
GQA-expanded ``[B, Hq, T, D]`` after ``repeat_kv``).
"""
from __future__ import annotations

import math
import os
from enum import Enum
from typing import List, Optional, Tuple

import torch


def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """``pace/llm/models/llama.py:50-61``: query head ``h`` reads KV head ``h // n_rep``."""
    if n_rep == 1:
        return x
    return torch.repeat_interleave(x, n_rep, dim=1)


class CacheKind(Enum):
    """``pace/llm/cache.py:18-33`` (``KVCacheType``)."""

    DYNAMIC = "dynamic"
    BMC = "bmc"

    @staticmethod
    def parse(kind) -> "CacheKind":
        return CacheKind(kind) if isinstance(kind, str) else kind


class _ContiguousCacheRef:
    """State shared by both caches (``pace/llm/cache.py:126-167``)."""

    def __init__(self) -> None:
        self.key: Optional[torch.Tensor] = None
        self.value: Optional[torch.Tensor] = None
        self.seq_len = 0
        self.concat_dim: Optional[int] = None

    def _pin_concat_dim(self, concat_dim: int) -> None:
        # cache.py:283-289 / 384-390: first call fixes the axis, later calls assert it.
        if self.concat_dim is None:
            self.concat_dim = concat_dim
        elif self.concat_dim != concat_dim:
            raise AssertionError("concat_dim should be the same for all updates")

    def _held(self) -> bool:
        return self.key is not None and self.value is not None

    def update_mask(self, attn_mask: torch.Tensor, input_size: int) -> torch.Tensor:
        """``cache.py:152-159``: identity unless overridden."""
        return attn_mask

    def update_cache_with_beam_indices(self, beam_idx: torch.Tensor) -> None:
        """``cache.py:161-167``: batch-row gather into fresh storage."""
        if self._held():
            self.key = torch.index_select(self.key, 0, beam_idx)
            self.value = torch.index_select(self.value, 0, beam_idx)

    def _check_remove(self, remove_len: int) -> None:
        if remove_len > self.seq_len:
            raise ValueError("Cannot remove more tokens than available in cache.")


class DynamicKVCacheRef(_ContiguousCacheRef):
    """``cache.py:329-400``: grows by concatenation, shrinks by re-narrowing."""

    def __init__(self, max_seq_length: int) -> None:
        super().__init__()

    def update_cache(self, key_states, value_states, concat_dim: int):
        self._pin_concat_dim(concat_dim)
        if self._held():
            self.key = torch.cat((self.key, key_states), dim=concat_dim)
            self.value = torch.cat((self.value, value_states), dim=concat_dim)
        else:  # first call keeps the caller's tensors by reference (cache.py:396-398)
            self.key, self.value = key_states, value_states
        self.seq_len = int(self.key.size(concat_dim))
        return self.key, self.value

    def remove_cache(self, remove_len: int) -> None:
        """``cache.py:352-368``."""
        if not self._held():
            return
        self._check_remove(remove_len)
        self.seq_len -= remove_len
        self.key = self.key.narrow(self.concat_dim, 0, self.seq_len)
        self.value = self.value.narrow(self.concat_dim, 0, self.seq_len)


class BMCKVCacheRef(_ContiguousCacheRef):
    """``cache.py:170-326``: zero-padded buffer re-allocated in ``tokens_per_split`` steps."""

    def __init__(self, max_seq_length: int) -> None:
        super().__init__()
        # cache.py:177-181: env override, else floor(sqrt(max_seq_length)) splits.
        splits = int(os.getenv("PACE_BMC_NUM_SPLITS", int(math.sqrt(max_seq_length))))
        self.tokens_per_split = max_seq_length // splits

    def capacity_for(self, n_tokens: int) -> int:
        """Padded length holding ``n_tokens`` (``cache.py:304-308``)."""
        return ((n_tokens - 1) // self.tokens_per_split + 1) * self.tokens_per_split

    def update_mask(self, attn_mask: torch.Tensor, input_size: int) -> torch.Tensor:
        """``cache.py:195-222``: right-pad the last axis with ``finfo.min`` up to capacity."""
        pad = self.capacity_for(input_size) - input_size
        shape = list(attn_mask.shape)
        shape[-1] = pad
        filler = torch.full(shape, torch.finfo(attn_mask.dtype).min, dtype=attn_mask.dtype)
        return torch.cat((attn_mask, filler), dim=-1)

    def remove_cache(self, remove_len: int) -> None:
        """``cache.py:224-240``: only the length moves; stale rows stay in the buffer."""
        if not self._held():
            return
        self._check_remove(remove_len)
        self.seq_len -= remove_len

    def update_cache(self, key_states, value_states, concat_dim: int):
        """``cache.py:242-326``."""
        self._pin_concat_dim(concat_dim)
        axis = self.concat_dim
        n_new = key_states.size(axis)
        total = self.seq_len + n_new
        # cache.py:296-301: note ">=" -- a buffer that would become exactly full is re-made.
        if not self._held() or total >= self.key.size(axis):
            shape = list(key_states.shape)
            shape[axis] = self.capacity_for(total)
            grown_k = torch.zeros(shape, dtype=key_states.dtype)
            grown_v = torch.zeros(shape, dtype=key_states.dtype)
            if self._held():  # cache.py:255-266: whole old buffer (stale rows too) into the prefix
                grown_k.narrow(axis, 0, self.key.size(axis)).copy_(self.key)
                grown_v.narrow(axis, 0, self.value.size(axis)).copy_(self.value)
            self.key, self.value = grown_k, grown_v
        self.key.narrow(axis, self.seq_len, n_new).copy_(key_states)
        self.value.narrow(axis, self.seq_len, value_states.size(concat_dim)).copy_(value_states)
        self.seq_len = total
        return self.key, self.value


def cache_class_for(kind):
    """``cache.py:36-45``."""
    kind = CacheKind.parse(kind)
    if kind is CacheKind.DYNAMIC:
        return DynamicKVCacheRef
    if kind is CacheKind.BMC:
        return BMCKVCacheRef
    raise ValueError(f"Invalid cache type: {kind}")


class KVCacheManagerRef:
    """``cache.py:48-123``: one cache per layer, one shared length."""

    def __init__(self, config, max_seq_length: int, cache_type) -> None:
        self.num_layers = config.num_hidden_layers
        self.cache_type = cache_type
        cls = cache_class_for(cache_type)
        self.cache_objects: List[_ContiguousCacheRef] = [
            cls(max_seq_length) for _ in range(self.num_layers)
        ]

    def __len__(self) -> int:
        return int(self.cache_objects[0].seq_len)

    def __getitem__(self, idx: int):
        return self.cache_objects[idx]

    def update_mask(self, attn_mask, input_size: int):
        return self.cache_objects[0].update_mask(attn_mask, input_size)

    def update_cache_with_beam_indices(self, beam_idx) -> None:
        for c in self.cache_objects:
            c.update_cache_with_beam_indices(beam_idx)

    def remove_cache(self, remove_len: int) -> None:
        for c in self.cache_objects:
            c.remove_cache(remove_len)


def valid_prefix(cache: _ContiguousCacheRef) -> Tuple[torch.Tensor, torch.Tensor]:
    """The live ``[.., :seq_len, ..]`` rows of a cache (drops BMC padding / stale rows)."""
    return (
        cache.key.narrow(cache.concat_dim, 0, cache.seq_len),
        cache.value.narrow(cache.concat_dim, 0, cache.seq_len),
    )
