"""KV-cache manager interface of the reference, backed by block-paged HBM storage.

Interface kept from ``pace/llm/cache.py`` of the reference:

* ``KVCacheType`` (``:18-33``) -- string-constructible enum, plus ``PAGED``.
* ``KVCacheManager(config, max_seq_length, cache_type)`` (``:48-123``) -- one cache
  per ``config.num_hidden_layers``; ``len()``, ``[]``, ``update_mask``,
  ``update_cache_with_beam_indices``, ``remove_cache``.
* ``KVCacheBase`` (``:126-167``) -- ``update_cache(key_states, value_states,
  concat_dim) -> (key, value)``, ``remove_cache(remove_len)``, ``update_mask``,
  ``update_cache_with_beam_indices``; attributes ``key``, ``value``, ``seq_len``,
  ``concat_dim``.

Error behaviour kept: changed ``concat_dim`` -> ``AssertionError``
(``:286-289``); over-long removal -> ``ValueError("Cannot remove more tokens
than available in cache.")`` (``:237-238``); unknown type -> ``ValueError``.

``PagedKVCache`` stores ``num_kv_heads`` heads (a GQA-expanded input, which is
what the reference's models pass after ``repeat_kv``, ``pace/llm/models/llama.py:151-158``,
is de-duplicated by stride) and returns *views* instead of dense tensors;
``MultiHeadAttention`` accepts those views, and ``view.dense()`` materialises the
reference-shaped ``[B, Hq, L, D]`` tensor.
"""
from __future__ import annotations

import ctypes
import math
from abc import ABC, abstractmethod
from enum import Enum
from typing import List, Optional, Sequence, Tuple, Union

import numpy as np
import torch

from .. import _native as nat
from ..utils.logging import PACE_LLM_ASSERT, PACE_LLM_DEBUG
from .paged import BLOCK, PagedState, blocks_for


class KVCacheType(Enum):
    DYNAMIC = "dynamic"
    BMC = "bmc"
    PAGED = "paged"

    @staticmethod
    def get_kv_cache_type(cache_type: Union[str, "KVCacheType"]) -> "KVCacheType":
        return KVCacheType(cache_type) if isinstance(cache_type, str) else cache_type


def get_kv_cache_class(cache_type: Union[str, KVCacheType]):
    cache_type = KVCacheType.get_kv_cache_type(cache_type)
    if cache_type is KVCacheType.PAGED:
        return PagedKVCache
    if cache_type in (KVCacheType.DYNAMIC, KVCacheType.BMC):
        from .contiguous import BMCKVCache, DynamicKVCache

        return DynamicKVCache if cache_type is KVCacheType.DYNAMIC else BMCKVCache
    raise ValueError(f"Invalid cache type: {cache_type}")


class KVCacheBase(ABC):
    """Per-layer cache contract (reference ``cache.py:126-167``)."""

    key = None
    value = None
    seq_len = 0
    concat_dim: Optional[int] = None

    @abstractmethod
    def update_cache(self, key_states, value_states, concat_dim: int):
        ...

    @abstractmethod
    def remove_cache(self, remove_len: int) -> None:
        ...

    def update_mask(self, attn_mask: torch.Tensor, input_size: int) -> torch.Tensor:
        return attn_mask

    def update_cache_with_beam_indices(self, beam_idx: torch.Tensor) -> None:
        if self.key is not None and self.value is not None:
            self.key = self.key.index_select(0, beam_idx.to(self.key.device))
            self.value = self.value.index_select(0, beam_idx.to(self.value.device))

    def _pin_concat_dim(self, concat_dim: int) -> None:
        if self.concat_dim is None:
            self.concat_dim = concat_dim
        else:
            PACE_LLM_ASSERT(self.concat_dim == concat_dim, "concat_dim should be the same for all updates")


class PagedKVView:
    """What ``PagedKVCache.update_cache`` returns in place of a dense tensor."""

    def __init__(self, cache: "PagedKVCache", which: str):
        self.cache = cache
        self.which = which

    @property
    def shape(self) -> Tuple[int, int, int, int]:
        c = self.cache
        return (c.batch, c.num_kv_heads * c.n_rep, int(c.lens.max(initial=0)), c.model_dim)

    def size(self, dim: int) -> int:
        return self.shape[dim]

    def dense(self, n_rep: Optional[int] = None, pad_to: Optional[int] = None) -> torch.Tensor:
        k, v = self.cache.gather(n_rep=n_rep, pad_to=pad_to)
        return k if self.which == "key" else v


class PagedKVCache(KVCacheBase):
    """One layer of block-paged K/V in HBM.

    ``shared`` lets the layers of a ``KVCacheManager`` use one block table.
    ``num_kv_heads`` (or ``n_rep``) tells the cache how a GQA-expanded input maps
    to stored heads; with neither, every input head is stored.
    """

    def __init__(
        self,
        max_seq_length: int,
        *,
        shared: Optional[dict] = None,
        num_kv_heads: Optional[int] = None,
        n_rep: Optional[int] = None,
        num_blocks: Optional[int] = None,
    ):
        self.max_seq_length = int(max_seq_length)
        self._shared = shared if shared is not None else {}
        self._cfg_kv_heads = num_kv_heads
        self._cfg_n_rep = n_rep
        self._cfg_num_blocks = num_blocks
        self.state: Optional[PagedState] = None
        self.pool: Optional[torch.Tensor] = None
        self._desc: Optional[nat.PoolDesc] = None
        self.lens = np.zeros(0, dtype=np.int64)
        self.seq_len = 0
        self.concat_dim = None
        self.key: Optional[PagedKVView] = None
        self.value: Optional[PagedKVView] = None
        self.batch = 0
        self.num_kv_heads = 0
        self.n_rep = 1
        self.head_dim = 0   # head size of the pool: one the kernels are built for
        self.model_dim = 0  # head size of the caller's tensors (smaller where it is not such a size: zero-padded)
        self.partition_tokens = 0  # 0: let the library choose
        # Appends of up to 32 tokens are held back until the attention call that follows, which
        # reads them from the caller's tensors and stores them into the pool in the same launch;
        # anything else that needs the pool or the lengths first flushes them with a plain append.
        self.fuse_append = True
        self._pending: Optional[Tuple[torch.Tensor, torch.Tensor, int, object]] = None
        self._query_rope = None
        self._graph = None  # a DecodeGraph that has captured this cache's decode step
        self.cow_blocks_copied = 0  # blocks copied on write after forks (per layer pool)
        self.f32 = False  # the pool holds fp32 rows (set by the first update)
        self._graph_appended = False  # fp32, inside a captured step: this step's append has been launched
        PACE_LLM_DEBUG(f"PagedKVCache initialized with max sequence length: {max_seq_length}")

    @property
    def lens(self) -> np.ndarray:
        """Tokens held per sequence (host copy)."""
        return self._lens

    @lens.setter
    def lens(self, value: np.ndarray) -> None:
        self._lens = value

    # -- set-up -----------------------------------------------------------------
    def _lazy_init(self, key_states: torch.Tensor) -> None:
        if self.pool is not None:
            return
        if not key_states.is_cuda:
            raise RuntimeError("PagedKVCache stores its blocks in GPU memory; key/value states must be device tensors")
        if key_states.dtype not in (torch.bfloat16, torch.float32):
            raise RuntimeError(f"PagedKVCache stores bf16 or fp32; got {key_states.dtype}")
        # fp32 (the reference's caches keep the model's dtype, ``pace/llm/cache.py:255-266``): blocks of plain rows,
        # read by the dense operator's fp32 kernel through the block table; the append rides in that launch when it
        # has up to 32 query rows per KV head (decode, short verify steps), the rotary embedding never does
        self.f32 = key_states.dtype == torch.float32
        nat.load()
        B, h_in, _, D = key_states.shape
        if self._cfg_kv_heads is not None:
            hkv = int(self._cfg_kv_heads)
        elif self._cfg_n_rep is not None:
            hkv = h_in // int(self._cfg_n_rep)
        else:
            hkv = h_in
        if h_in % hkv:
            raise RuntimeError(f"{h_in} input heads cannot be reduced to {hkv} KV heads")
        self.batch, self.num_kv_heads, self.model_dim = int(B), hkv, int(D)
        # e.g. 80 (OPT-2.7B) is kept in slabs of 96: zero dims change neither a score nor an output
        self.head_dim = (D + 3) // 4 * 4 if self.f32 else next((d for d in nat.HEAD_DIMS if d >= D), 0)
        if not self.head_dim or self.head_dim > nat.HEAD_DIMS[-1]:
            raise RuntimeError(f"head_dim {D} unsupported (at most {nat.HEAD_DIMS[-1]})")
        D = self.head_dim
        self.n_rep = int(self._cfg_n_rep) if self._cfg_n_rep is not None else h_in // hkv
        if "state" not in self._shared:
            self._shared["state"] = PagedState(B, self.max_seq_length, self._cfg_num_blocks, key_states.device)
        self.state = self._shared["state"]
        if self.state.batch != B:
            raise RuntimeError(f"batch changed from {self.state.batch} to {B}")
        nb = self.state.allocator.num_blocks
        # [block][head][K|V][16*D]: one block of one layer is contiguous (64 KiB at 8 heads x 128 dims)
        # and the K and V slabs a wavefront reads together are adjacent.
        self.pool = torch.zeros((nb, hkv, 2, BLOCK * D), dtype=key_states.dtype, device=key_states.device)
        self.state.pools.append(self.pool)
        self._desc = self._describe(self.pool)
        self.state.pool_descs.append(self._desc)
        self.lens = np.zeros(B, dtype=np.int64)

    def _describe(self, pool: torch.Tensor) -> nat.PoolDesc:
        nb, hkv, _, slab = pool.shape
        return nat.PoolDesc(
            k=pool[:, :, 0].data_ptr(),
            v=pool[:, :, 1].data_ptr(),
            k_block_stride=pool.stride(0),
            k_head_stride=pool.stride(1),
            v_block_stride=pool.stride(0),
            v_head_stride=pool.stride(1),
            num_blocks=nb,
            num_kv_heads=hkv,
            head_dim=slab // BLOCK,
            block_size=BLOCK,
            elem_bytes=pool.element_size(),
        )

    # -- reference interface ----------------------------------------------------
    def update_cache(self, key_states: torch.Tensor, value_states: torch.Tensor, concat_dim: int, rope=None):
        """Append ``T`` tokens to every sequence (reference ``cache.py:268-326``).

        ``rope`` (what ``RotaryEmbedding.forward`` returned for this step) hands over the
        *un-rotated* keys: they are rotated on their way into the pool, and the attention
        call that follows rotates its *un-rotated* queries the same way -- the
        rope / repeat_kv / update_cache / attention sequence of
        ``pace/llm/models/llama.py:147-165`` as one launch for steps of up to 32 tokens.
        """
        self._pin_concat_dim(concat_dim)
        PACE_LLM_ASSERT(key_states.dim() == 4 and concat_dim == 2, "PagedKVCache expects [B, H, T, D] with concat_dim=2")
        self._lazy_init(key_states)
        self._append(key_states, value_states, None, rope)
        return self.key, self.value

    def remove_cache(self, remove_len: int) -> None:
        """Drop the last ``remove_len`` tokens of every sequence (reference ``cache.py:224-240``)."""
        if self.pool is None:
            return
        if remove_len > self.seq_len or (self.lens < remove_len).any():
            raise ValueError("Cannot remove more tokens than available in cache.")
        self.truncate(np.full(self.batch, int(remove_len), dtype=np.int64))

    def update_cache_with_beam_indices(self, beam_idx: torch.Tensor) -> None:
        """Batch-row gather (reference ``cache.py:161-167``): sequence ``i`` becomes a
        copy of old sequence ``beam_idx[i]``; blocks are copied on the device."""
        if self.pool is None:
            return
        self.reorder([int(i) for i in beam_idx.tolist()])

    # -- paged-only surface -----------------------------------------------------
    def append_ragged(self, key_states: torch.Tensor, value_states: torch.Tensor, counts: Sequence[int],
                      right_aligned: bool = False):
        """Append ``counts[b]`` of the ``T`` given tokens to sequence ``b``: the first ones of its
        row, or with ``right_aligned`` the last ones (the alignment multi-token attention uses for
        its query rows, so a ragged verify step passes q, k and v padded the same way)."""
        self._pin_concat_dim(2)
        self._lazy_init(key_states)
        self._append(key_states, value_states, np.asarray(counts, dtype=np.int64), right_aligned=right_aligned)
        return self.key, self.value

    def _append(self, k: torch.Tensor, v: torch.Tensor, counts: Optional[np.ndarray], rope=None,
                right_aligned: bool = False) -> None:
        B, h_in, T, D = k.shape
        if rope is not None and (counts is not None or tuple(rope.rows.shape) not in ((B, T), (1, T))):
            raise RuntimeError("rope rows must be [B, T] (or [1, T]) and cannot be combined with per-sequence counts")
        if B != self.batch or D != self.model_dim or h_in % self.num_kv_heads:
            raise RuntimeError(f"update of shape {tuple(k.shape)} does not fit cache [B={self.batch}, Hkv={self.num_kv_heads}, D={D}]")
        if v.shape != k.shape:
            raise RuntimeError("key_states and value_states differ in shape")
        if self.head_dim != self.model_dim:
            # (a rotary embedding then rotates the first rotary_dim <= model_dim dims of the padded rows, in a launch of
            # its own: inside the attention launch it needs rotary_dim == the pool's head size)
            k, v = (torch.nn.functional.pad(t, (0, self.head_dim - self.model_dim)) for t in (k, v))
        if k.dtype != self.pool.dtype or v.dtype != self.pool.dtype:
            raise RuntimeError(f"the cache holds {self.pool.dtype}; got {k.dtype} / {v.dtype}")
        ks = k.stride()
        per16 = 4 if self.f32 else 8  # elements in 16 bytes
        if ks[3] != 1 or ks != v.stride() or ks[0] % per16 or ks[1] % per16 or ks[2] % per16:
            k, v = k.contiguous(), v.contiguous()
        if self.f32 and rope is not None:
            # rotated in a launch of its own; the attention call that follows does the same with its queries
            _, k = rope(None, k)
            self._query_rope, rope = rope, None
            keep_query_rope = True
        else:
            keep_query_rope = False
        head_step = h_in // self.num_kv_heads  # de-duplicate a repeat_kv-expanded input
        st = self.state
        lib = nat.load()
        if (self._graph is not None and counts is None and (self.fuse_append or self.f32) and T <= 32
                and self._pending is None and not self._graph_appended):
            # a step of a decode graph: blocks and table were prepared for every step, and the lengths advance on the
            # device.  The append rides in the attention launch; over an fp32 pool only with up to 32 query rows per KV
            # head (else, or with fuse_append off: a launch of its own, its positions taken from the graph's frozen
            # lengths plus the device counter).
            graph = self._graph
            graph.reserve(T)
            if self.f32 and (not self.fuse_append or T * self.n_rep > 32):
                nat.check(
                    lib.pace_kv_append_paged_at(
                        ctypes.byref(self._desc), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1) * head_step, k.stride(2),
                        B, T, graph.table.data_ptr(), graph.table.stride(0), graph.lens_dev.data_ptr(), 0,
                        graph.counter.data_ptr(), nat.current_stream_ptr(),
                    )
                )
                self._graph_appended = True
                if not keep_query_rope:
                    self._query_rope = None
            else:
                self._pending = (k, v, head_step, rope)
                self._query_rope = rope
            self.lens = self.lens + T
            self.seq_len += T
            return
        self._flush()
        if st.tails_dirty:
            self._unshare()
        if counts is None:
            new_lens = self.lens + T
            if self.seq_len + T > st.min_capacity:
                st.ensure_capacity(new_lens)
            if self.fuse_append and T <= 32:
                self._pending = (k, v, head_step, rope)
            else:
                self._launch_append(k, v, head_step, new_lens, rope)
            if not keep_query_rope:
                self._query_rope = rope  # the next attention call rotates its queries with it
        else:
            if (counts < 0).any() or (counts > T).any():
                raise ValueError("counts must lie in [0, T]")
            new_lens = self.lens + counts
            st.ensure_capacity(new_lens)
            slots = torch.from_numpy(st.slots(self.lens, counts, T, right_aligned)).pin_memory().to(k.device, non_blocking=True)
            nat.check(
                lib.pace_kv_append(
                    ctypes.byref(self._desc), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1) * head_step, k.stride(2),
                    B, T, slots.data_ptr(), nat.current_stream_ptr(),
                )
            )
        self.lens = new_lens
        self.seq_len = self.seq_len + T if counts is None else int(new_lens.max(initial=0))
        if self.key is None:
            self.key, self.value = PagedKVView(self, "key"), PagedKVView(self, "value")

    def _launch_append(self, k: torch.Tensor, v: torch.Tensor, head_step: int, lens_after: np.ndarray, rope=None) -> None:
        st = self.state
        T = k.shape[2]
        (lens_dev, bias), table = st.device_lens(lens_after), st.device_table()
        if rope is not None:
            desc = rope.desc()
            nat.check(
                nat.load().pace_rope_append_paged(
                    ctypes.byref(self._desc), ctypes.byref(desc), None, None, 0, 0, 0, 0,
                    k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1) * head_step, k.stride(2),
                    self.batch, T, table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias - T, nat.current_stream_ptr(),
                )
            )
            return
        nat.check(
            nat.load().pace_kv_append_paged(
                ctypes.byref(self._desc), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1) * head_step, k.stride(2),
                self.batch, T, table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias - T, nat.current_stream_ptr(),
            )
        )

    def _flush(self) -> None:
        """Store a held-back append into the pool now.  Every operation other than a captured decode step
        comes through here first, which ends a decode graph (its frozen plan and lengths no longer hold)."""
        if self._graph is not None:
            if self._graph._capturing:
                # anything that comes through here uploads host data or allocates blocks: recorded into a graph it
                # would replay stale values
                raise RuntimeError("the captured step differs from its eager run: a cache operation other than the "
                                   "step's one update_cache + attention per layer ran during the capture")
            self._graph.close()
        self._graph_appended = False
        if self._pending is not None:
            k, v, head_step, rope = self._pending
            self._pending = None
            self._launch_append(k, v, head_step, self.lens, rope)

    def truncate(self, remove: Sequence[int]) -> None:
        """Per-sequence rollback: forget the last ``remove[b]`` tokens of sequence ``b``
        and return emptied blocks to the free list."""
        self._flush()
        remove = np.asarray(remove, dtype=np.int64)
        if (remove > self.lens).any() or (remove < 0).any():
            raise ValueError("Cannot remove more tokens than available in cache.")
        self.lens = self.lens - remove
        self.seq_len = int(self.lens.max(initial=0))
        if remove.any():
            self._release()
            self.state.lengths_shrank()

    def _release(self) -> None:
        # Blocks are shared by every layer: only the longest view of a sequence frees.
        peers = self._shared.get("layers")
        lens = self.lens if not peers else np.max([p.lens for p in peers if p.pool is not None], axis=0)
        self.state.release_beyond(lens)

    def evict_blocks(self, b: int, logical_blocks: Sequence[int]) -> None:
        """Remove whole logical blocks from the middle of sequence ``b``; the
        surviving tokens keep their order and become the sequence."""
        peers = [p for p in self._shared.get("layers", [self]) if p.pool is not None]
        for p in peers:
            p._flush()
        new_lens = self.state.evict(b, logical_blocks, self.lens)
        self.state.lengths_shrank()
        for p in peers:
            p.lens = new_lens.copy()
            p.seq_len = int(new_lens.max(initial=0))

    def compact(self) -> int:
        """Pack live blocks into the lowest pool ids (every layer's pool); returns blocks moved."""
        for p in self._shared.get("layers", [self]):
            if p.pool is not None:
                p._flush()
        # one library call plans the moves, uploads them and starts the copies of every layer's pool
        moves = self.state.compact_blocks(self.state.pool_descs)
        if len(moves):
            self.state.apply_moves(moves)  # the table rewrite runs on the host while the GPU copies
        return len(moves)

    def reorder(self, beam_idx: Sequence[int]) -> None:
        """Sequence ``i`` becomes old sequence ``beam_idx[i]``.  No K/V moves here: the block
        tables are re-pointed and the blocks get several owners; the one block per sequence that
        the next append writes into is copied then (copy-on-write, ``_unshare``)."""
        st = self.state
        peers = [p for p in self._shared.get("layers", [self]) if p.pool is not None]
        for p in peers:
            p._flush()
        src = [int(i) for i in beam_idx]
        st.fork(src)
        for p in peers:
            p.lens = p.lens[src].copy()
            p.seq_len = int(p.lens.max(initial=0))

    def _unshare(self) -> None:
        """Give every sequence a private copy of the block its next token lands in (all layers)."""
        st = self.state
        peers = [p for p in self._shared.get("layers", [self]) if p.pool is not None]
        for p in peers:
            p._flush()
        lens = np.min([p.lens for p in peers], axis=0)  # the earliest position any layer will write
        pairs = st.unshare_tails(lens)
        if len(pairs):
            dev = st.upload_pairs(pairs)
            lib = nat.load()
            for pool in st.pools:
                desc = self._describe(pool)
                nat.check(lib.pace_kv_copy_blocks(ctypes.byref(desc), ctypes.byref(desc), dev.data_ptr(), len(pairs), nat.current_stream_ptr()))
        self.cow_blocks_copied += len(pairs)

    def gather(self, n_rep: Optional[int] = None, pad_to: Optional[int] = None,
               zero_fill: bool = True) -> Tuple[torch.Tensor, torch.Tensor]:
        """Dense ``[B, Hkv*n_rep, L, D]`` copies of K and V, zeros past each length (what the
        reference's caches hold, ``pace/llm/cache.py:255-266``).  ``zero_fill=False`` leaves the rows
        past each length unwritten: in a ragged batch they are most of the tensor."""
        self._flush()
        n_rep = self.n_rep if n_rep is None else int(n_rep)
        L = int(self.lens.max(initial=0)) if pad_to is None else int(pad_to)
        shape = (self.batch, self.num_kv_heads * n_rep, L, self.head_dim)
        padded = self.head_dim != self.model_dim
        k = torch.empty(shape, dtype=self.pool.dtype, device=self.pool.device)
        v = torch.empty(shape, dtype=self.pool.dtype, device=self.pool.device)
        if L:
            st = self.state
            table, (lens_dev, bias) = st.device_table(), st.device_lens(self.lens)
            total = int(self.lens.sum())
            if not zero_fill and 0 < total < 1 << 31:
                # nothing to write past the lengths: one workgroup per block that exists (in a ragged batch most of
                # the [B, L] row range is padding)
                cu = np.zeros(self.batch + 1, dtype=np.int64)
                np.cumsum(self.lens, out=cu[1:])
                cu_dev = torch.from_numpy(cu.astype(np.int32)).pin_memory().to(self.pool.device, non_blocking=True)
                nat.check(
                    nat.load().pace_kv_gather_live(
                        ctypes.byref(self._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias, cu_dev.data_ptr(),
                        self.batch, n_rep, k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), L, total, nat.current_stream_ptr(),
                    )
                )
            elif zero_fill or total:
                nat.check(
                    nat.load().pace_kv_gather(
                        ctypes.byref(self._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias, self.batch, n_rep,
                        k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), L, 1 if zero_fill else 0, nat.current_stream_ptr(),
                    )
                )
        if padded:
            k, v = k[..., : self.model_dim].contiguous(), v[..., : self.model_dim].contiguous()
        return k, v

    def gather_packed(self, n_rep: Optional[int] = None) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        """K and V without padding: ``[sum(lens), Hkv*n_rep, D]`` each, the rows of sequence ``b`` at
        ``cu_seqlens[b] : cu_seqlens[b+1]`` (third result, device int32 ``[B+1]``).  Row ``t`` of
        sequence ``b`` is ``dense[b, :, t, :]``."""
        self._flush()
        n_rep = self.n_rep if n_rep is None else int(n_rep)
        cu = np.zeros(self.batch + 1, dtype=np.int64)
        np.cumsum(self.lens, out=cu[1:])
        total = int(cu[-1])
        if total >= 1 << 31:
            raise RuntimeError("packed gather addresses rows with 32-bit offsets")
        dev = self.pool.device
        cu_dev = torch.from_numpy(cu.astype(np.int32)).pin_memory().to(dev, non_blocking=True)
        shape = (total, self.num_kv_heads * n_rep, self.head_dim)
        k = torch.empty(shape, dtype=self.pool.dtype, device=dev)
        v = torch.empty(shape, dtype=self.pool.dtype, device=dev)
        if total:
            st = self.state
            table, (lens_dev, bias) = st.device_table(), st.device_lens(self.lens)
            nat.check(
                nat.load().pace_kv_gather_packed(
                    ctypes.byref(self._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias, cu_dev.data_ptr(),
                    self.batch, n_rep, k.data_ptr(), v.data_ptr(), total, nat.current_stream_ptr(),
                )
            )
        if self.head_dim != self.model_dim:
            k, v = k[..., : self.model_dim].contiguous(), v[..., : self.model_dim].contiguous()
        return k, v, cu_dev

    def attend(self, query: torch.Tensor, attention_mask: Optional[torch.Tensor] = None,
               kv_start: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``softmax(q K^T / sqrt(D) + mask) V`` of ``query [B, Hq, S, D]`` over this cache.

        Without a mask, row ``s`` of sequence ``b`` reads tokens ``<= len_b - S + s``
        (the causal mask ``pace/llm/models/llama.py:292-299`` builds); with an additive
        mask ``[B|1, 1, S|1, Lm]`` the mask alone decides, as in the reference.
        """
        if query.dim() != 4 or not query.is_cuda or self.pool is None or query.dtype != self.pool.dtype:
            raise RuntimeError("paged attention expects a device tensor [B, Hq, S, D] of the cache's dtype (bf16 or fp32)")
        B, hq, S, D = query.shape
        if B != self.batch or D != self.model_dim or hq % self.num_kv_heads:
            raise RuntimeError(f"query {tuple(query.shape)} does not fit cache [B={self.batch}, Hkv={self.num_kv_heads}, D={self.model_dim}]")
        if self.head_dim != self.model_dim:
            query, D = torch.nn.functional.pad(query, (0, self.head_dim - self.model_dim)), self.head_dim
        qs = query.stride()
        per16 = 4 if self.f32 else 8
        if qs[3] != 1 or qs[0] % per16 or qs[1] % per16 or qs[2] % per16 or query.data_ptr() % 16:
            query = query.contiguous()
            qs = query.stride()
        if self.f32 and self._pending is not None and self._graph is None and S * (hq // self.num_kv_heads) > 32:
            self._flush()  # over an fp32 pool the append rides in launches of up to 32 query rows per KV head
        rope, self._query_rope = self._query_rope, None
        rope_desc = None
        if rope is not None:
            if tuple(rope.rows.shape) not in ((B, S), (1, S)):
                raise RuntimeError(f"rope rows {tuple(rope.rows.shape)} do not match the query [B={B}, S={S}]")
            rope_desc = None if self.f32 else rope.desc()
            if self.f32:
                query, _ = rope(query, None)  # (the keys were rotated before their append)
                qs = query.stride()
            elif attention_mask is not None or rope_desc.rotary_dim != D:
                # cases the attention launch does not fold in: rotate the queries (and a held-back append) first
                self._flush()
                query, _ = rope(query, None)
                qs = query.stride()
                rope_desc = None
        out = torch.empty((B, hq, S, D), dtype=query.dtype, device=query.device)
        st = self.state
        max_len = self.seq_len
        lib = nat.load()
        graph = self._graph
        if graph is not None and self._pending is None and not self._graph_appended:
            if graph._capturing:
                raise RuntimeError("the captured step differs from its eager run: attention without the step's append")
            graph.close()  # attention without the step's append is not the captured step
            graph = None
        self._graph_appended = False
        plan = lambda: st.plan_attention(self.lens, hq, self.num_kv_heads, self.head_dim, S, attention_mask is not None,
                                         self.partition_tokens)
        a = nat.PagedAttnArgs()
        if self.f32:
            # rows of fp32: one launch of the dense operator's kernel over the block table, no work list, no workspace
            items = parts = None
            n_items = max_parts = ws_bytes = 0
            rows = S * (hq // self.num_kv_heads)
            if B * self.num_kv_heads * ((rows + 63) // 64 if rows > 32 else 1) < 512:
                # a batch that does not fill the GPU: room for the library to cut every sequence over up to 64 workgroups
                ws_bytes = min(B * hq * S * 64 * (D + 4) * 4, 64 << 20)
            if graph is None:
                table, (lens_dev, bias) = st.device_table(), st.device_lens(self.lens)
                a.seq_len_bias = bias
            else:  # captured step: frozen table and lengths, the device counter counts the tokens of the steps before
                table, lens_dev = graph.table, graph.lens_dev
                a.seq_len_bias, a.seq_len_bias_ptr = graph.new_tokens, graph.counter.data_ptr()
                max_len = int(graph.base.max()) + graph.new_tokens * graph.max_steps
        elif graph is None:
            items, parts, n_items, max_parts, ws_bytes = plan()
            table, (lens_dev, bias) = st.device_table(), st.device_lens(self.lens)
            a.seq_len_bias = bias
        else:
            # captured step: the plan and the table are frozen, the lengths are base + new tokens + the device counter
            items, parts, n_items, max_parts, ws_bytes = graph.plan((hq, S, attention_mask is not None), plan)
            table, lens_dev = graph.table, graph.lens_dev
            a.seq_len_bias, a.seq_len_bias_ptr = graph.new_tokens, graph.counter.data_ptr()
            max_len = int(graph.base.max()) + graph.new_tokens * graph.max_steps
        ws = st.workspace(ws_bytes)
        a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = query.data_ptr(), qs[0], qs[1], qs[2]
        a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = out.data_ptr(), hq * S * D, S * D, D  # (allocated above: contiguous)
        a.block_table, a.table_stride = table.data_ptr(), table.stride(0)
        a.seq_lens = lens_dev.data_ptr()
        a.kv_start = None if kv_start is None else kv_start.data_ptr()
        if attention_mask is not None:
            m = attention_mask
            if m.dim() != 4 or m.size(1) != 1 or m.size(0) not in (1, B) or m.size(2) not in (1, S):
                raise RuntimeError(f"paged attention takes a mask [B|1, 1, S|1, L]; got {tuple(m.shape)}")
            if m.dtype not in (torch.float32, torch.bfloat16):
                raise RuntimeError("pace::SDPA attention only support the dtypes Float and BF16 types for input Attention mask")
            if m.stride(3) != 1:
                m = m.contiguous()
            a.mask = m.data_ptr()
            a.mask_dtype = nat.DTYPE_F32 if m.dtype == torch.float32 else nat.DTYPE_BF16
            a.mask_len = m.size(3)
            a.mask_stride_b = 0 if m.size(0) == 1 else m.stride(0)
            a.mask_stride_s = 0 if m.size(2) == 1 else m.stride(2)
            a.causal = 0
        else:
            a.mask, a.causal = None, 1
        a.batch, a.num_q_heads, a.q_len = B, hq, S
        a.max_seq_len, a.partition_tokens = max_len, 0
        if items is not None:
            a.work_items, a.n_work_items = items.data_ptr(), n_items
            a.seq_parts, a.max_parts = parts.data_ptr(), max_parts
        a.scale = 1.0 / math.sqrt(self.model_dim)
        a.workspace = None if ws is None else ws.data_ptr()
        a.workspace_bytes = ws_bytes
        if rope_desc is not None:
            a.rope = ctypes.pointer(rope_desc)
        if self._pending is not None:
            k, v, head_step, k_rope = self._pending
            if (k_rope is None) != (rope_desc is None) or k.shape[2] != S and rope_desc is not None:
                raise RuntimeError("a held-back append and the attention call disagree about the rotary embedding")
            self._pending = None  # this launch stores them into the pool
            ks = k.stride()
            a.k_new, a.v_new, a.n_new = k.data_ptr(), v.data_ptr(), k.shape[2]
            a.new_stride_b, a.new_stride_h, a.new_stride_t = ks[0], ks[1] * head_step, ks[2]
        fn = lib.pace_paged_attn_decode if S == 1 else lib.pace_paged_attn_verify
        nat.check(fn(ctypes.byref(self._desc), ctypes.byref(a), nat.current_stream_ptr()))
        return out if self.head_dim == self.model_dim else out[..., : self.model_dim].contiguous()


class KVCacheManager:
    """One cache per layer, one shared length (reference ``cache.py:48-123``).

    For ``KVCacheType.PAGED`` the layers share one block table; ``num_kv_heads``
    is taken from ``config.num_key_value_heads`` when the config has it, so the
    GQA-expanded K/V the reference's models pass in are stored once per KV head.
    """

    def __init__(self, config, max_seq_length: int, cache_type: Union[str, KVCacheType], **paged_options):
        self.num_layers = config.num_hidden_layers
        self.cache_type = cache_type
        self.kv_cache_class = get_kv_cache_class(cache_type)
        if self.kv_cache_class is PagedKVCache:
            shared: dict = {}
            opts = dict(paged_options)
            opts.setdefault("num_kv_heads", getattr(config, "num_key_value_heads", None))
            heads = getattr(config, "num_attention_heads", None)
            if heads and opts["num_kv_heads"]:
                opts.setdefault("n_rep", heads // opts["num_kv_heads"])
            self.cache_objects: List[KVCacheBase] = [
                PagedKVCache(max_seq_length, shared=shared, **opts) for _ in range(self.num_layers)
            ]
            shared["layers"] = self.cache_objects
        else:
            self.cache_objects = [self.kv_cache_class(max_seq_length) for _ in range(self.num_layers)]

    def __len__(self) -> int:
        return int(self.cache_objects[0].seq_len)

    def __getitem__(self, idx: int) -> KVCacheBase:
        return self.cache_objects[idx]

    def update_mask(self, attn_mask: torch.Tensor, input_size: int) -> torch.Tensor:
        return self.cache_objects[0].update_mask(attn_mask, input_size)

    def update_cache_with_beam_indices(self, beam_idx: torch.Tensor) -> None:
        if self.kv_cache_class is PagedKVCache:
            self.cache_objects[0].update_cache_with_beam_indices(beam_idx)  # moves every layer's blocks
            return
        for cache_object in self.cache_objects:
            cache_object.update_cache_with_beam_indices(beam_idx)

    def remove_cache(self, remove_len: int) -> None:
        for cache_object in self.cache_objects:
            cache_object.remove_cache(remove_len)

    def capture_decode(self, step_fn, max_steps: int):
        """Capture one decode step over every layer into a HIP graph (paged caches only): see
        ``pace_mi355.llm.graph.DecodeGraph``.  ``step_fn`` runs the step on static tensors; the returned
        object's ``replay()`` runs it again for the next token."""
        if self.kv_cache_class is not PagedKVCache:
            raise RuntimeError("only the paged cache keeps its lengths on the device; capture_decode needs KVCacheType.PAGED")
        from .graph import DecodeGraph

        return DecodeGraph(list(self.cache_objects), step_fn, max_steps)
