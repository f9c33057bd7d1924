"""Oracle: contiguous-semantics model of the block-paged cache operations.

TEST INFRASTRUCTURE -- see ``oracle/__init__.py``.

The reference has no paged storage.  Every paged operation of the product is a
permutation of token rows, so its expected result is stated on the reference's
*contiguous* cache: per sequence, the rows the reference's ``DynamicKVCache``
(``pace/llm/cache.py:370-400``) would hold had it been fed only the surviving
tokens, in order.  ``RaggedCacheModel`` keeps exactly that, one tensor per
sequence; ``dense()`` lays it out as the reference does
(``[B, Hq, L, D]`` after ``repeat_kv``, ``pace/llm/models/llama.py:151-158``).

``scatter_slots`` / ``gather_slots`` / ``copy_blocks_np`` state the slot-level
semantics on a logical ``[num_slots, Hkv, D]`` row table with numpy indexing
(``numpy.take`` / fancy assignment are the library routines that pin them).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from .attention_ref import lengths_mask_4d, sdpa_fp32
from .cache_ref import repeat_kv


class RaggedCacheModel:
    """One layer of K/V rows per sequence, ``[Hkv, len_b, D]`` each."""

    def __init__(self, batch: int, num_kv_heads: int, head_dim: int, dtype=torch.bfloat16):
        self.dtype = dtype
        self.k: List[torch.Tensor] = [torch.zeros(num_kv_heads, 0, head_dim, dtype=dtype) for _ in range(batch)]
        self.v: List[torch.Tensor] = [torch.zeros(num_kv_heads, 0, head_dim, dtype=dtype) for _ in range(batch)]

    @property
    def batch(self) -> int:
        return len(self.k)

    def seq_lens(self) -> List[int]:
        return [int(t.shape[1]) for t in self.k]

    def append(self, k_new: torch.Tensor, v_new: torch.Tensor, counts: Optional[Sequence[int]] = None) -> None:
        """Append ``k_new[b, :, :counts[b]]`` to sequence ``b`` (``cache.py:391-395``: ``torch.cat``)."""
        for b in range(self.batch):
            n = k_new.shape[2] if counts is None else int(counts[b])
            self.k[b] = torch.cat((self.k[b], k_new[b, :, :n].to(self.dtype)), dim=1)
            self.v[b] = torch.cat((self.v[b], v_new[b, :, :n].to(self.dtype)), dim=1)

    def truncate(self, remove: Sequence[int]) -> None:
        """Per-sequence suffix removal; one sequence of it is ``cache.py:352-368``."""
        for b, r in enumerate(remove):
            r = int(r)
            if r > self.k[b].shape[1]:
                raise ValueError("Cannot remove more tokens than available in cache.")
            keep = self.k[b].shape[1] - r
            self.k[b] = self.k[b][:, :keep]
            self.v[b] = self.v[b][:, :keep]

    def evict_blocks(self, b: int, logical_blocks: Sequence[int], block_size: int) -> None:
        """Drop the token rows of the given logical blocks of sequence ``b``;
        survivors keep their order (what a cache fed only the survivors holds)."""
        n = self.k[b].shape[1]
        keep = np.ones(n, dtype=bool)
        for j in logical_blocks:
            keep[j * block_size : min((j + 1) * block_size, n)] = False
        idx = torch.from_numpy(np.nonzero(keep)[0])
        self.k[b] = self.k[b].index_select(1, idx)
        self.v[b] = self.v[b].index_select(1, idx)

    def reorder(self, beam_idx: Sequence[int]) -> None:
        """Batch-row gather (``cache.py:161-167``)."""
        self.k = [self.k[int(i)].clone() for i in beam_idx]
        self.v = [self.v[int(i)].clone() for i in beam_idx]

    def dense(self, n_rep: int = 1, pad_to: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor]:
        """Zero-right-padded ``[B, Hkv*n_rep, L, D]`` pair, heads expanded as ``repeat_kv``."""
        lens = self.seq_lens()
        L = max(lens + [0]) if pad_to is None else pad_to
        H, _, D = self.k[0].shape
        K = torch.zeros(self.batch, H, L, D, dtype=self.dtype)
        V = torch.zeros(self.batch, H, L, D, dtype=self.dtype)
        for b, n in enumerate(lens):
            K[b, :, :n] = self.k[b]
            V[b, :, :n] = self.v[b]
        return repeat_kv(K, n_rep), repeat_kv(V, n_rep)

    def attention(self, q: torch.Tensor, n_rep: int, causal_tail: bool = True) -> torch.Tensor:
        """fp32 reference attention of ``q [B, Hq, S, D]`` over the cache.

        Query row ``s`` of sequence ``b`` sits at position ``len_b - S + s`` and
        reads tokens ``<=`` its position: the mask ``llama.py:292-299`` builds
        for ``S`` new tokens on top of ``len_b - S`` cached ones.
        """
        K, V = self.dense(n_rep)
        S = q.shape[2]
        mask = lengths_mask_4d(self.seq_lens(), S if causal_tail else 1, K.shape[2], torch.float32)
        if not causal_tail and S > 1:
            mask = mask.expand(-1, -1, S, -1)
        return sdpa_fp32(q, K, V, mask)


# ---- slot-level semantics on a logical row table ---------------------------------


def scatter_slots(rows: np.ndarray, new_rows: np.ndarray, slots: np.ndarray) -> None:
    """``rows[slots[i]] = new_rows[i]`` for ``slots[i] >= 0`` (negative = padding, skipped)."""
    live = slots >= 0
    rows[slots[live]] = new_rows[live]


def slots_for(block_table: np.ndarray, b: int, start: int, count: int, block_size: int) -> np.ndarray:
    """Slot ids of tokens ``start .. start+count-1`` of sequence ``b``."""
    pos = np.arange(start, start + count)
    return block_table[b, pos // block_size].astype(np.int64) * block_size + pos % block_size


def gather_slots(rows: np.ndarray, block_table: np.ndarray, seq_lens: Sequence[int], block_size: int, pad_to: int) -> np.ndarray:
    """Dense ``[B, pad_to, ...]`` view of each sequence's rows, zero beyond its length."""
    out = np.zeros((len(seq_lens), pad_to) + rows.shape[1:], dtype=rows.dtype)
    for b, n in enumerate(seq_lens):
        out[b, :n] = np.take(rows, slots_for(block_table, b, 0, int(n), block_size), axis=0)
    return out


def copy_blocks_np(pool: np.ndarray, pairs: np.ndarray) -> None:
    """``pool[dst] = pool[src]`` for each ``(src, dst)`` row of ``pairs``; the
    source and destination id sets must be disjoint (so order is irrelevant)."""
    src, dst = pairs[:, 0], pairs[:, 1]
    assert not (set(src.tolist()) & set(dst.tolist()))
    pool[dst] = pool[src]
