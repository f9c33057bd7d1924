"""Host-side bookkeeping of the block-paged KV store: free list, block tables,
per-sequence lengths, device mirrors, and the plans for eviction / compaction.

The reference has no paged storage (its caches are contiguous tensors,
``pace/llm/cache.py:170-400``); this module is the new surface behind the
reference's ``KVCacheBase`` interface.  All arithmetic here is integer
bookkeeping on the host; every byte of K/V moves in the HIP kernels.
"""
from __future__ import annotations

from typing import Iterable, List, Optional, Sequence, Tuple

import ctypes

import numpy as np
import torch

from .. import _native as nat

BLOCK = nat.BLOCK_TOKENS


def blocks_for(n_tokens: int) -> int:
    return (int(n_tokens) + BLOCK - 1) // BLOCK


class BlockAllocator:
    """LIFO free list over pool block ids ``0 .. num_blocks-1`` (lowest ids first), with a
    reference count per block: sequences forked from one another (beam search) point at the
    same blocks until one of them writes.  The free list is a stack in a numpy array (its top at
    ``_n_free``), so allocation, release and wholesale rebuilds cost no per-block interpreter work."""

    def __init__(self, num_blocks: int):
        self.num_blocks = int(num_blocks)
        self._stack = np.arange(self.num_blocks - 1, -1, -1, dtype=np.int32)
        self._n_free = self.num_blocks
        self._is_free = np.ones(self.num_blocks, dtype=bool)
        self.refs = np.zeros(self.num_blocks, dtype=np.int32)
        self._order = np.zeros(self.num_blocks, dtype=np.int32)  # scratch of free_in_turn

    @property
    def num_free(self) -> int:
        return self._n_free

    def allocate(self, n: int) -> List[int]:
        return self.allocate_array(n).tolist()

    def allocate_array(self, n: int) -> np.ndarray:
        """``n`` blocks off the top of the stack, in the order ``n`` single allocations would hand them out."""
        if n > self._n_free:
            raise MemoryError(f"KV block pool exhausted: need {n} blocks, {self._n_free} free of {self.num_blocks}")
        if n == 0:
            return np.zeros(0, dtype=np.int32)
        out = self._stack[self._n_free - n:self._n_free][::-1].copy()
        self._n_free -= n
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
        arr = np.asarray(ids if isinstance(ids, np.ndarray) else list(ids), dtype=np.int64)
        if not arr.size:
            return
        if self._is_free[arr].any():
            raise ValueError(f"block {int(arr[self._is_free[arr]][0])} freed twice")
        np.subtract.at(self.refs, arr, 1)
        if (self.refs[arr] < 0).any():
            raise ValueError(f"block {int(arr[self.refs[arr] < 0][0])} freed twice")
        gone = arr[self.refs[arr] == 0]
        if gone.size:
            _, first = np.unique(gone, return_index=True)  # an id listed twice is pushed once, in order of appearance
            gone = gone[np.sort(first)]
            self._is_free[gone] = True
            self._stack[self._n_free:self._n_free + gone.size] = gone
            self._n_free += gone.size

    def free_in_turn(self, arr: np.ndarray) -> None:
        """``free`` of each id of ``arr`` one after the other, in one go: a block that loses several owners here
        returns to the free list where its last owner drops it."""
        arr = np.asarray(arr, dtype=np.int64)
        if not arr.size:
            return
        if self._is_free[arr].any():
            raise ValueError(f"block {int(arr[self._is_free[arr]][0])} freed twice")
        if (self.refs[arr] == 1).all():
            # no block here has another owner (the usual case: no forked sequences): each returns as it is listed.
            # An id listed twice would be a block freed twice: the second write of its position shows it.
            self._order[arr] = np.arange(arr.size, dtype=np.int32)
            if (self._order[arr] != np.arange(arr.size, dtype=np.int32)).any():
                raise ValueError("a block with one owner freed twice")
            self.refs[arr] = 0
            gone = arr
        else:
            np.subtract.at(self.refs, arr, 1)
            if (self.refs[arr] < 0).any():
                raise ValueError(f"block {int(arr[self.refs[arr] < 0][0])} freed twice")
            gone = arr[self.refs[arr] == 0]
            if gone.size:
                _, last = np.unique(gone[::-1], return_index=True)  # an id listed twice is pushed once, where it occurs last
                gone = gone[np.sort(gone.size - 1 - last)]
        if gone.size:
            self._is_free[gone] = True
            self._stack[self._n_free:self._n_free + gone.size] = gone
            self._n_free += gone.size

    def take(self, ids: Iterable[int]) -> None:
        """Mark specific ids as used (compaction destinations)."""
        want = np.unique(np.asarray(list(ids), dtype=np.int64))
        if want.size and not self._is_free[want].all():
            raise ValueError(f"block {int(want[~self._is_free[want]][0])} is not free")
        self._is_free[want] = False
        self.refs[want] = 1
        keep = self._stack[:self._n_free]
        keep = keep[self._is_free[keep]]
        self._stack[:keep.size] = keep
        self._n_free = keep.size

    def reset_free(self, is_free: np.ndarray, refs: Optional[np.ndarray] = None) -> None:
        """Replace the free list wholesale (lowest ids are handed out first again)."""
        self._is_free = is_free.copy()
        free = np.nonzero(is_free)[0][::-1]
        self._stack[:free.size] = free
        self._n_free = free.size
        self.refs = refs.astype(np.int32) if refs is not None else (~is_free).astype(np.int32)

    def free_ids(self) -> np.ndarray:
        return np.nonzero(self._is_free)[0]

    def free_flags_ptr(self) -> int:
        """Address of the free flags, one byte per block id (1 = free), for the native planner."""
        assert self._is_free.dtype == np.bool_ and self._is_free.flags.c_contiguous
        return self._is_free.ctypes.data


def _ragged_cells(first: np.ndarray, count: np.ndarray) -> Tuple[np.ndarray, np.ndarray]:
    """Row and column indices of cells ``first[b] .. first[b] + count[b] - 1`` of every row ``b``, row by row."""
    count = np.asarray(count, dtype=np.int64)
    rows = np.repeat(np.arange(count.size), count)
    starts = np.cumsum(count) - count
    cols = np.arange(int(count.sum())) - np.repeat(starts, count) + np.repeat(np.asarray(first, dtype=np.int64), count)
    return rows, cols


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
        self.pool_descs: list = []  # the library's descriptor of each pool, in the same order
        self._table_dev: Optional[torch.Tensor] = None
        self._table_dirty = True
        self._lens_dev: Optional[torch.Tensor] = None
        self._lens_host: Optional[np.ndarray] = None
        self._workspace: Optional[torch.Tensor] = None
        self.min_capacity = 0  # tokens every sequence can hold in the blocks it already owns
        self.has_shared = False  # some block has more than one owner (after a fork)
        self.tails_dirty = False  # a sequence's last, partly filled block may have other owners
        self.table_version = 0  # bumped when table entries below the sequences' lengths change (not by appends)
        self._items_key = None
        self._items_dev: Optional[torch.Tensor] = None
        self._parts_dev: Optional[torch.Tensor] = None
        self._items_host: Optional[torch.Tensor] = None
        self._items_dev_buf: Optional[torch.Tensor] = None
        self._items_copied = None
        self._pairs_host: Optional[torch.Tensor] = None
        self._pairs_dev: Optional[torch.Tensor] = None
        self._pairs_copied = None
        self._pairs_event = None
        self._n_items, self._max_parts, self._plan_ws = 0, 1, 0

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
        grow = np.maximum(need - self.n_blocks, 0)
        total = int(grow.sum())
        if total:
            # every sequence's new blocks in one allocation, in the order one allocation per sequence would give them
            rows, cols = _ragged_cells(self.n_blocks, grow)
            self.table[rows, cols] = self.allocator.allocate_array(total)
            self.n_blocks = np.maximum(self.n_blocks, need).astype(self.n_blocks.dtype)
            self._table_dirty = True
        self.min_capacity = self._min_blocks() * BLOCK

    def release_beyond(self, lens: np.ndarray) -> int:
        """Free the blocks no token of ``lens`` touches any more; returns how many."""
        need = (lens + BLOCK - 1) // BLOCK
        drop = np.maximum(self.n_blocks - need, 0)
        freed = int(drop.sum())
        if freed:
            rows, cols = _ragged_cells(np.minimum(self.n_blocks, need), drop)
            self.allocator.free_in_turn(self.table[rows, cols])
            self.table[rows, cols] = 0
            self.n_blocks = np.minimum(self.n_blocks, need).astype(self.n_blocks.dtype)
            self._table_dirty = True
        if freed:
            self.table_version += 1
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
        self.table_version += 1
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
                self.table_version += 1
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

    def plan_attention(self, lens: np.ndarray, num_q_heads: int, num_kv_heads: int, head_dim: int, q_len: int,
                       masked: bool, partition_tokens: int):
        """Work list of one attention launch over sequences of ``lens`` tokens (new tokens included).

        Returns ``(items, seq_parts, n_items, max_parts, workspace_bytes)``: ``items`` is the device ``int32
        [n_items][16]`` descriptor list ``pace_paged_attn_plan`` wrote (the cut of every sequence into
        partitions, in scheduling order, with the pool blocks of each partition's first units), ``seq_parts``
        the device ``int32 [B]`` partition counts.  A plan is kept while the lengths stay in the same 64-token
        buckets and no table entry below them changed: appends in between grow the last partition of each
        sequence, which the kernels follow from the device-side lengths.
        """
        key = (self.table_version, num_q_heads, num_kv_heads, head_dim, q_len, bool(masked), partition_tokens,
               (lens // 64).tobytes())
        if key == self._items_key:
            return self._items_dev, self._parts_dev, self._n_items, self._max_parts, self._plan_ws
        B = self.batch
        lens32 = np.ascontiguousarray(lens, dtype=np.int32)
        cap = int(((lens32 + 31) // 32).sum()) + B  # most work items there can be: a partition holds a unit or more
        if self._items_host is None or self._items_host.shape[0] < cap + B:
            size = max(2 * cap, 64) + B
            pin = self.device.type == "cuda"
            self._items_copied = None
            self._items_host = torch.empty((size, nat.WORK_INTS), dtype=torch.int32, pin_memory=pin)
            self._items_dev_buf = torch.empty((size, nat.WORK_INTS), dtype=torch.int32, device=self.device)
        host = self._items_host
        if self._items_copied is not None:
            self._items_copied.synchronize()  # the upload of the plan before this one has read the staging buffer
        # row 0 .. : descriptors; the partition counts ride behind them in the same buffer (one upload)
        plan = nat.AttnPlan()
        parts_row = host.shape[0] - (B + nat.WORK_INTS - 1) // nat.WORK_INTS
        parts_ptr = host.data_ptr() + parts_row * nat.WORK_INTS * 4
        nat.check(nat.load().pace_paged_attn_plan(
            lens32.ctypes.data, self.table.ctypes.data, self.table.shape[1], B, num_q_heads, num_kv_heads, head_dim, q_len,
            1 if masked else 0, partition_tokens, host.data_ptr(), parts_row, parts_ptr, ctypes.byref(plan)))
        n = int(plan.n_work_items)
        dev = self._items_dev_buf
        if self.device.type == "cuda":
            dev[:n].copy_(host[:n], non_blocking=True)
            dev[parts_row:].copy_(host[parts_row:], non_blocking=True)
            self._items_copied = torch.cuda.Event()
            self._items_copied.record()
        else:
            dev = host
        self._items_dev = dev[:n]
        self._parts_dev = dev[parts_row:].view(-1)[:B]
        self._n_items, self._max_parts, self._plan_ws = n, int(plan.max_parts), int(plan.workspace_bytes)
        self._items_key = key
        return self._items_dev, self._parts_dev, n, self._max_parts, self._plan_ws

    def upload_pairs(self, pairs: np.ndarray) -> torch.Tensor:
        """Device copy of an ``int32 [n][2]`` list of (src, dst) blocks, through a pinned staging buffer that
        is kept (allocating pinned memory costs more than the copy of a few thousand pairs)."""
        n = len(pairs)
        if self.device.type != "cuda":
            return torch.from_numpy(np.ascontiguousarray(pairs, dtype=np.int32))
        if self._pairs_host is None or self._pairs_host.shape[0] < n:
            size = max(1024, 2 * n)
            self._pairs_copied = None
            self._pairs_host = torch.empty((size, 2), dtype=torch.int32, pin_memory=True)
            self._pairs_dev = torch.empty((size, 2), dtype=torch.int32, device=self.device)
        if self._pairs_copied is not None:
            self._pairs_copied.synchronize()  # the upload before this one has read the staging buffer
        self._pairs_host.numpy()[:n] = pairs
        self._pairs_dev[:n].copy_(self._pairs_host[:n], non_blocking=True)
        self._pairs_copied = torch.cuda.Event()
        self._pairs_copied.record()
        return self._pairs_dev[:n]

    def compact_blocks(self, descs) -> np.ndarray:
        """Plan the compaction, upload its moves and start the block copies of every pool in ``descs`` (pool
        descriptors that share this table) with one library call; returns the moves ``[n][2]`` (a view of the pinned
        staging buffer: valid until the next upload).  The table is not rewritten here: ``apply_moves`` does
        that on the host while the copies run."""
        cap = self.allocator.num_blocks
        if self._pairs_host is None or self._pairs_host.shape[0] < cap:
            self._pairs_copied = None
            self._pairs_host = torch.empty((cap, 2), dtype=torch.int32, pin_memory=True)
            self._pairs_dev = torch.empty((cap, 2), dtype=torch.int32, device=self.device)
        if self._pairs_copied is not None:
            self._pairs_copied.synchronize()  # the upload before this one has read the staging buffer
        ptrs = (ctypes.c_void_p * len(descs))(*[ctypes.addressof(d) for d in descs])
        n = int(nat.load().pace_kv_compact_blocks(
            ptrs, len(descs), self.table.ctypes.data, self.table.shape[1], self.n_blocks.ctypes.data, self.batch,
            self.allocator.free_flags_ptr(), self._pairs_host.data_ptr(), cap, self._pairs_dev.data_ptr(), nat.current_stream_ptr()))
        if n < 0:
            nat.check(n)
        if n:
            if self._pairs_event is None:
                self._pairs_event = torch.cuda.Event()
            self._pairs_event.record()
            self._pairs_copied = self._pairs_event
        return self._pairs_host.numpy()[:n]

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
        self.table_version += 1
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
        sets are disjoint.  (The passes over the table run in the library.)"""
        moves = np.empty((self.allocator.num_blocks, 2), dtype=np.int32)
        n = int(nat.load().pace_kv_plan_compaction_flags(self.allocator.free_flags_ptr(), self.allocator.num_blocks, moves.ctypes.data,
                                                         moves.shape[0]))
        if n < 0:
            nat.check(n)
        return moves[:n]

    def apply_moves(self, moves: np.ndarray) -> None:
        """Rewrite the tables and the free list for ``moves`` (whose data the caller copies; the copy may
        still be running: nothing here touches the device)."""
        if not len(moves):
            return
        moves = np.ascontiguousarray(moves, dtype=np.int32)
        alloc = self.allocator
        n_free = ctypes.c_int32(0)
        # the table, the owners per block, the free flags and the free list in one pass of native code
        nat.check(nat.load().pace_kv_apply_moves_tracked(
            self.table.ctypes.data, self.table.shape[1], self.n_blocks.ctypes.data, self.batch, alloc.num_blocks,
            moves.ctypes.data, len(moves), alloc.refs.ctypes.data, alloc.free_flags_ptr(), alloc._stack.ctypes.data, ctypes.byref(n_free)))
        alloc._n_free = int(n_free.value)
        self._table_dirty = True
        self.table_version += 1

    def live_block_count(self) -> int:
        """Pool blocks in use (a block with several owners counts once)."""
        return int((self.allocator.refs > 0).sum())
