"""Host-side bookkeeping of the block-paged KV store: free list, block tables,
per-sequence lengths, device mirrors, and the plans for eviction / compaction.

The reference has no paged storage (its caches are contiguous tensors,
``pace/llm/cache.py:170-400``); this module is the new surface behind the
reference's ``KVCacheBase`` interface.  All arithmetic here is integer
bookkeeping on the host; every byte of K/V moves in the HIP kernels.
"""
from __future__ import annotations

from typing import Iterable, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import _native as nat

BLOCK = nat.BLOCK_TOKENS


def blocks_for(n_tokens: int) -> int:
    return (int(n_tokens) + BLOCK - 1) // BLOCK


class BlockAllocator:
    """LIFO free list over pool block ids ``0 .. num_blocks-1`` (lowest ids first), with a
    reference count per block: sequences forked from one another (beam search) point at the
    same blocks until one of them writes."""

    def __init__(self, num_blocks: int):
        self.num_blocks = int(num_blocks)
        self._free: List[int] = list(range(self.num_blocks - 1, -1, -1))
        self._is_free = np.ones(self.num_blocks, dtype=bool)
        self.refs = np.zeros(self.num_blocks, dtype=np.int32)

    @property
    def num_free(self) -> int:
        return len(self._free)

    def allocate(self, n: int) -> List[int]:
        if n > len(self._free):
            raise MemoryError(f"KV block pool exhausted: need {n} blocks, {len(self._free)} free of {self.num_blocks}")
        if n == 0:
            return []
        out = self._free[-n:][::-1]
        del self._free[-n:]
        self._is_free[out] = False
        self.refs[out] = 1
        return out

    def share(self, ids: Iterable[int]) -> None:
        """One more owner for each of ``ids`` (an id may occur several times)."""
        ids = np.asarray(list(ids), dtype=np.int64)
        if ids.size:
            if self._is_free[ids].any():
                raise ValueError("cannot share a free block")
            np.add.at(self.refs, ids, 1)

    def free(self, ids: Iterable[int]) -> None:
        """Drop one owner of each of ``ids``; a block returns to the free list with its last owner."""
        ids = [int(i) for i in ids]
        if not ids:
            return
        arr = np.asarray(ids, dtype=np.int64)
        if self._is_free[arr].any():
            raise ValueError(f"block {[i for i in ids if self._is_free[i]][0]} freed twice")
        np.subtract.at(self.refs, arr, 1)
        if (self.refs[arr] < 0).any():
            raise ValueError(f"block {[i for i in ids if self.refs[i] < 0][0]} freed twice")
        gone = [i for i in dict.fromkeys(ids) if self.refs[i] == 0]
        if gone:
            self._is_free[gone] = True
            self._free.extend(gone)

    def take(self, ids: Iterable[int]) -> None:
        """Mark specific ids as used (compaction destinations)."""
        want = set(int(i) for i in ids)
        for i in want:
            if not self._is_free[i]:
                raise ValueError(f"block {i} is not free")
            self._is_free[i] = False
            self.refs[i] = 1
        self._free = [i for i in self._free if i not in want]

    def reset_free(self, is_free: np.ndarray, refs: Optional[np.ndarray] = None) -> None:
        """Replace the free list wholesale (lowest ids are handed out first again)."""
        self._is_free = is_free.copy()
        self._free = np.nonzero(is_free)[0][::-1].tolist()
        self.refs = refs.astype(np.int32) if refs is not None else (~is_free).astype(np.int32)

    def free_ids(self) -> np.ndarray:
        return np.nonzero(self._is_free)[0]


class PagedState:
    """Block tables and lengths of one batch, shared by every layer's pool.

    All layers append the same tokens at the same positions, so one block table
    serves them all (block ``i`` of every layer's pool belongs to the same
    sequence range).  Lengths are tracked per call site: a layer passes the
    lengths it is at, and the device mirror is refreshed only when they differ
    from what the device already holds.
    """

    def __init__(self, batch: int, max_seq_length: int, num_blocks: Optional[int], device: torch.device):
        self.batch = int(batch)
        self.device = device
        self.max_blocks_per_seq = max(1, blocks_for(max_seq_length))
        if num_blocks is None:
            num_blocks = self.batch * self.max_blocks_per_seq
        self.allocator = BlockAllocator(num_blocks)
        self.table = np.zeros((self.batch, self.max_blocks_per_seq), dtype=np.int32)
        self.n_blocks = np.zeros(self.batch, dtype=np.int64)  # table entries in use per sequence
        self.pools: List["torch.Tensor"] = []  # one [num_blocks][Hkv][2][16*D] tensor per layer
        self._table_dev: Optional[torch.Tensor] = None
        self._table_dirty = True
        self._lens_dev: Optional[torch.Tensor] = None
        self._lens_host: Optional[np.ndarray] = None
        self._workspace: Optional[torch.Tensor] = None
        self.min_capacity = 0  # tokens every sequence can hold in the blocks it already owns
        self.has_shared = False  # some block has more than one owner (after a fork)
        self.tails_dirty = False  # a sequence's last, partly filled block may have other owners
        self._items_key = None
        self._items_dev: Optional[torch.Tensor] = None
        self._parts_dev: Optional[torch.Tensor] = None
        self._max_parts = 1

    # -- capacity ---------------------------------------------------------------
    def _min_blocks(self) -> int:
        return int(self.n_blocks.min()) if self.n_blocks.size else 0

    def _grow_table(self, need_cols: int) -> None:
        if need_cols <= self.table.shape[1]:
            return
        cols = max(need_cols, 2 * self.table.shape[1])
        grown = np.zeros((self.batch, cols), dtype=np.int32)
        grown[:, : self.table.shape[1]] = self.table
        self.table = grown
        self._table_dirty = True
        self._table_dev = None

    def ensure_capacity(self, lens: np.ndarray) -> None:
        """Give every sequence enough blocks to hold ``lens[b]`` tokens."""
        need = (lens + BLOCK - 1) // BLOCK
        self._grow_table(int(need.max(initial=0)))
        for b in np.nonzero(need > self.n_blocks)[0]:
            have, want = int(self.n_blocks[b]), int(need[b])
            self.table[b, have:want] = self.allocator.allocate(want - have)
            self.n_blocks[b] = want
            self._table_dirty = True
        self.min_capacity = self._min_blocks() * BLOCK

    def release_beyond(self, lens: np.ndarray) -> int:
        """Free the blocks no token of ``lens`` touches any more; returns how many."""
        need = (lens + BLOCK - 1) // BLOCK
        freed = 0
        for b in np.nonzero(need < self.n_blocks)[0]:
            have, want = int(self.n_blocks[b]), int(need[b])
            self.allocator.free(self.table[b, want:have].tolist())
            self.table[b, want:have] = 0
            self.n_blocks[b] = want
            freed += have - want
            self._table_dirty = True
        if freed:
            self.min_capacity = self._min_blocks() * BLOCK
        return freed

    def lengths_shrank(self) -> None:
        """A rollback or an eviction can make a block with several owners the last block of a
        sequence again: the next append has to look at the tails once more."""
        if self.has_shared:
            self.has_shared = bool((self.allocator.refs > 1).any())
            self.tails_dirty = self.has_shared

    # -- forks (beam search) ----------------------------------------------------
    def fork(self, source_rows: Sequence[int]) -> None:
        """Sequence ``i`` becomes a copy of old sequence ``source_rows[i]`` without moving a byte:
        the new table rows point at the same blocks, which then have several owners.  The block a
        later append would write into is copied first (``unshare_tails``)."""
        src = [int(i) for i in source_rows]
        if len(src) != self.batch or any(i < 0 or i >= self.batch for i in src):
            raise IndexError(f"fork expects {self.batch} source rows in [0, {self.batch})")
        old_table, old_n = self.table.copy(), self.n_blocks.copy()
        for i in src:  # new owners first, so that no block is freed in between
            self.allocator.share(old_table[i, : int(old_n[i])].tolist())
        for b in range(self.batch):
            self.allocator.free(old_table[b, : int(old_n[b])].tolist())
        self.table[:] = 0
        for i, srow in enumerate(src):
            n = int(old_n[srow])
            self.table[i, :n] = old_table[srow, :n]
            self.n_blocks[i] = n
        self.has_shared = bool((self.allocator.refs > 1).any())
        self.tails_dirty = self.has_shared
        self._table_dirty = True
        self.min_capacity = self._min_blocks() * BLOCK

    def unshare_tails(self, lens: np.ndarray) -> np.ndarray:
        """Copy-on-write before an append at positions ``lens[b] ..``: a partly filled last block
        that has other owners is replaced by a fresh block.  Returns the ``(src, dst)`` pairs whose
        data the caller must copy (in every layer's pool) before anything is written."""
        pairs: List[Tuple[int, int]] = []
        self.tails_dirty = False
        if not self.has_shared:
            return np.zeros((0, 2), np.int32)
        for b in range(self.batch):
            pos = int(lens[b])
            jb = pos // BLOCK
            if pos % BLOCK == 0 or jb >= int(self.n_blocks[b]):
                continue  # the append starts a block of its own
            old = int(self.table[b, jb])
            if self.allocator.refs[old] > 1:
                new = self.allocator.allocate(1)[0]
                self.allocator.free([old])
                self.table[b, jb] = new
                pairs.append((old, new))
                self._table_dirty = True
        self.has_shared = bool((self.allocator.refs > 1).any())
        return np.asarray(pairs, dtype=np.int32).reshape(-1, 2)

    # -- device mirrors ---------------------------------------------------------
    def device_table(self) -> torch.Tensor:
        if self._table_dev is None or self._table_dirty:
            host = torch.from_numpy(self.table)
            if self._table_dev is None or self._table_dev.shape != host.shape:
                self._table_dev = torch.empty(host.shape, dtype=torch.int32, device=self.device)
            self._table_dev.copy_(host.pin_memory(), non_blocking=True)
            self._table_dirty = False
        return self._table_dev

    def device_lens(self, lens: np.ndarray) -> Tuple[torch.Tensor, int]:
        """``(tensor, bias)`` with ``tensor[b] + bias == lens[b]``: the int32 device mirror is only
        rewritten when the lengths stop being a uniform shift of what it holds (the kernels add
        the bias themselves)."""
        if self._lens_dev is not None:
            delta = lens - self._lens_host
            d0 = int(delta[0]) if delta.size else 0
            if (delta == d0).all():
                return self._lens_dev, d0
        host = torch.from_numpy(lens.astype(np.int32))
        if self._lens_dev is None:
            self._lens_dev = torch.empty(self.batch, dtype=torch.int32, device=self.device)
        self._lens_dev.copy_(host.pin_memory(), non_blocking=True)
        self._lens_host = lens.copy()
        return self._lens_dev, 0

    def plan_attention(self, lens: np.ndarray, part_tokens: int, part_cap: int, slots: int):
        """How to cut the sequences of a batch for one attention launch.

        Returns ``(items, seq_parts, max_parts)``: ``items`` is a device ``int32 [n][2]`` list of
        (sequence, partition) pairs, longest partitions first, or ``None`` when a dense grid has no
        empty entries (equal lengths, one partition rule).  ``seq_parts`` (device ``int32 [B]``) is
        set when the whole launch fits the GPU in one round: the partition counts are then chosen
        so that the partitions are as equal as possible and fill the ``slots`` workgroup slots
        (largest-remainder apportionment), instead of all sequences being cut at one length.
        """
        if lens.size == 0:
            return None, None, 1
        base = np.maximum(1, -(-lens // part_tokens))
        uniform = bool((lens == lens[0]).all())
        cap_parts = np.maximum(1, -(-lens // part_cap))
        if not uniform and int(cap_parts.sum()) < slots and int(base.sum()) <= slots:
            key = ("even", part_cap, slots, (lens // 64).tobytes())
            if key != self._items_key:
                n = cap_parts.copy()
                size = lens / n
                while int(n.sum()) < slots:
                    b = int(np.argmax(size))
                    if lens[b] / (n[b] + 1) < 256:
                        break
                    n[b] += 1
                    size[b] = lens[b] / n[b]
                self._store_items(key, lens, n, with_parts=True)
            return self._items_dev, self._parts_dev, self._max_parts
        if uniform:
            return None, None, int(base.max())
        key = ("cut", part_tokens, base.tobytes(), np.argsort(-lens, kind="stable")[:8].tobytes())
        if key != self._items_key:
            self._store_items(key, lens, base, with_parts=False)
        return self._items_dev, None, int(base.max())

    def _upload(self, host: torch.Tensor) -> torch.Tensor:
        """Asynchronous copy to the device through fresh pinned memory (plain tensor on a CPU state)."""
        if self.device.type != "cuda":
            return host
        return host.pin_memory().to(self.device, non_blocking=True)

    def _store_items(self, key, lens: np.ndarray, n_parts: np.ndarray, with_parts: bool) -> None:
        seq = np.repeat(np.arange(lens.size), n_parts)
        first = np.repeat(np.cumsum(n_parts) - n_parts, n_parts)
        part = np.arange(seq.size) - first
        size = np.repeat(lens / n_parts, n_parts)
        order = np.argsort(-size, kind="stable")
        items = np.stack([seq, part], axis=1)[order].astype(np.int32)
        self._items_dev = self._upload(torch.from_numpy(items))
        self._parts_dev = self._upload(torch.from_numpy(n_parts.astype(np.int32))) if with_parts else None
        self._max_parts = int(n_parts.max())
        self._items_key = key

    def workspace(self, nbytes: int) -> Optional[torch.Tensor]:
        if nbytes == 0:
            return None
        if self._workspace is None or self._workspace.numel() < nbytes:
            self._workspace = torch.empty(nbytes, dtype=torch.uint8, device=self.device)
        return self._workspace

    # -- slot arithmetic --------------------------------------------------------
    def slots(self, starts: np.ndarray, counts: np.ndarray, width: int, right_aligned: bool = False) -> np.ndarray:
        """``[B, width]`` int64 slot ids of tokens ``starts[b] .. starts[b]+counts[b]-1``; -1 pads.
        The ``counts[b]`` tokens of a row are its first ones, or its last ones with ``right_aligned``."""
        out = np.full((self.batch, width), -1, dtype=np.int64)
        for b in range(self.batch):
            n = int(counts[b])
            if n:
                pos = np.arange(int(starts[b]), int(starts[b]) + n)
                ids = self.table[b, pos // BLOCK].astype(np.int64) * BLOCK + pos % BLOCK
                if right_aligned:
                    out[b, width - n:] = ids
                else:
                    out[b, :n] = ids
        return out

    # -- block-level plans ------------------------------------------------------
    def evict(self, b: int, logical_blocks: Sequence[int], lens: np.ndarray) -> np.ndarray:
        """Drop the given logical blocks of sequence ``b``: their pool blocks go
        back to the free list, later table entries shift left, and the length
        shrinks by the tokens those blocks held.  Returns the new lengths."""
        n = int(self.n_blocks[b])
        drop = sorted(set(int(j) for j in logical_blocks))
        if drop and (drop[0] < 0 or drop[-1] >= n):
            raise IndexError(f"sequence {b} has {n} blocks; cannot evict {drop}")
        removed_tokens = sum(min(BLOCK, int(lens[b]) - j * BLOCK) for j in drop)
        keep = [j for j in range(n) if j not in set(drop)]
        self.allocator.free(self.table[b, drop].tolist())
        row = self.table[b, keep].copy()
        self.table[b, :] = 0
        self.table[b, : len(keep)] = row
        self.n_blocks[b] = len(keep)
        self._table_dirty = True
        self.min_capacity = self._min_blocks() * BLOCK
        out = lens.copy()
        out[b] -= removed_tokens
        return out

    def _live_mask(self) -> np.ndarray:
        """``[B, cols]`` bool: the table entries in use."""
        return np.arange(self.table.shape[1])[None, :] < self.n_blocks[:, None]

    def plan_compaction(self) -> np.ndarray:
        """Moves that pack all live blocks into ids ``0 .. n_live-1`` with the
        fewest copies: every live block at or above ``n_live`` moves into a free
        id below it.  Returns ``[n_moves, 2]`` int32 ``(src, dst)``; the two id
        sets are disjoint."""
        is_live = np.zeros(self.allocator.num_blocks, dtype=bool)
        is_live[self.table[self._live_mask()]] = True
        n_live = int(is_live.sum())
        src = np.nonzero(is_live[n_live:])[0] + n_live
        dst = np.nonzero(~is_live[:n_live])[0]
        assert src.size == dst.size
        return np.stack([src, dst], axis=1).astype(np.int32) if src.size else np.zeros((0, 2), np.int32)

    def apply_moves(self, moves: np.ndarray) -> None:
        """Rewrite the tables and the free list after the data of ``moves`` was copied."""
        if not len(moves):
            return
        remap = np.arange(self.allocator.num_blocks, dtype=np.int32)
        remap[moves[:, 0]] = moves[:, 1]
        mask = self._live_mask()
        self.table[mask] = remap[self.table[mask]]
        refs = np.bincount(self.table[mask], minlength=self.allocator.num_blocks).astype(np.int32)
        self.allocator.reset_free(refs == 0, refs)
        self._table_dirty = True

    def live_block_count(self) -> int:
        """Pool blocks in use (a block with several owners counts once)."""
        return int((self.allocator.refs > 0).sum())
