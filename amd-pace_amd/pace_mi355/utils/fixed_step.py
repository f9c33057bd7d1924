"""Set-up shared by the benchmark and the full-size parity tests: a paged cache filled with seeded data in a
seeded physical block order, and one step of the hot path issued straight through the C ABI with its metadata
frozen (the launch the headline figure is measured on)."""
from __future__ import annotations

import ctypes
import math

def randn_bf16(torch, shape, gen, dev):
    return torch.randn(*shape, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)


def build_cache(torch, dev, lens, q_heads, kv_heads, head_dim, seed, pool_factor=None, headroom=64, permute=True,
                history=False, f32=False):
    """Paged cache holding lens[b] tokens per sequence, physical blocks in a seeded random order (a shuffle of
    the free list) or, with `history`, in the order a seeded admit / retire history of sequences leaves behind."""
    import numpy as np
    from ..llm import PagedKVCache
    from .history import alloc_free_history

    B, T = len(lens), max(lens)
    live = sum((n + headroom + 15) // 16 for n in lens)
    num_blocks = int(pool_factor * live) if pool_factor else live
    cache = PagedKVCache(T + headroom, num_kv_heads=kv_heads, n_rep=q_heads // kv_heads, num_blocks=num_blocks)
    g = torch.Generator(device=dev).manual_seed(seed)
    lens_np = np.asarray(lens)
    chunk = 1024
    for t0 in range(0, T, chunk):
        n = min(chunk, T - t0)
        k = randn_bf16(torch, (B, kv_heads, n, head_dim), g, dev)
        v = randn_bf16(torch, (B, kv_heads, n, head_dim), g, dev)
        if f32:  # a pool of fp32 rows
            k, v = k.float(), v.float()
        if t0 == 0:
            cache.append_ragged(k[:, :, :1], v[:, :, :1], [0] * B)  # creates the pool and the free list
            alloc = cache.state.allocator
            if history:
                alloc_free_history(alloc, seed, 8, 1024)
                cache.append_ragged(k, v, np.clip(lens_np - t0, 0, n))
                continue
            ids = alloc.allocate(alloc.num_free)
            if permute:
                np.random.default_rng(seed).shuffle(ids)  # consecutive logical blocks end up far apart in HBM
            else:
                ids = ids[::-1]
            alloc.free(ids)
        cache.append_ragged(k, v, np.clip(lens_np - t0, 0, n))
    return cache


class FixedStep:
    """Direct C-ABI calls with metadata frozen at "T new tokens on top of the prefilled cache":
    the new tokens land on the same positions every step, so each step moves the same bytes."""

    def __init__(self, torch, cache, q, k_new, v_new, partition=0, fused=True, rope=None, mask=None):
        import numpy as np
        from .. import _native as nat

        self.nat, self.lib = nat, nat.load()
        dev = q.device
        B, hq, S, D = q.shape
        T = k_new.shape[2]
        self.cache, self.k, self.v, self.T, self.B = cache, k_new, v_new, T, B
        lens_after = cache.lens + T
        cache.state.ensure_capacity(lens_after)
        self.table = cache.state.device_table()
        self.lens_dev = torch.from_numpy(lens_after.astype(np.int32)).to(dev)
        self.lens_after = lens_after
        self.out = torch.empty(B, hq, S, D, dtype=q.dtype, device=dev)
        max_len = int(lens_after.max())
        a = nat.PagedAttnArgs()
        a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
        a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = (self.out.data_ptr(), self.out.stride(0), self.out.stride(1),
                                                           self.out.stride(2))
        a.block_table, a.table_stride, a.seq_lens = self.table.data_ptr(), self.table.stride(0), self.lens_dev.data_ptr()
        a.kv_start, a.mask, a.causal = None, None, 1
        if mask is not None:  # additive bf16 [B,1,S,L]: the mask alone decides what a row reads
            self.mask = mask
            a.mask, a.mask_dtype, a.mask_len, a.causal = mask.data_ptr(), nat.DTYPE_BF16, mask.shape[3], 0
            a.mask_stride_b, a.mask_stride_s = mask.stride(0), mask.stride(2)
        a.batch, a.num_q_heads, a.q_len = B, hq, S
        # the library's planner cuts the batch: descriptors of (sequence, partition) work items in scheduling order
        a.max_seq_len, a.partition_tokens, a.scale = max_len, 0, 1.0 / math.sqrt(D)
        if cache.f32:  # rows of fp32: one launch over the block table, no work list; the workspace lets a small batch be cut
            n_items = max_parts = 0
            ws_bytes = min(B * hq * S * 64 * (D + 4) * 4, 64 << 20)
        else:
            self.items, self.parts, n_items, max_parts, ws_bytes = cache.state.plan_attention(
                lens_after, hq, cache.num_kv_heads, cache.head_dim, S, mask is not None, partition)
            a.work_items, a.n_work_items = self.items.data_ptr(), n_items
            a.seq_parts, a.max_parts = self.parts.data_ptr(), max_parts
        self.ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        a.workspace, a.workspace_bytes = self.ws.data_ptr(), ws_bytes
        self.n_items, self.max_parts = n_items, max_parts
        self.fused = fused
        if fused:  # the attention launch reads the new tokens from k_new / v_new and stores them into the pool
            a.k_new, a.v_new, a.n_new = k_new.data_ptr(), v_new.data_ptr(), T
            a.new_stride_b, a.new_stride_h, a.new_stride_t = k_new.stride(0), k_new.stride(1), k_new.stride(2)
        # rope (a pace_rope_t with positions == NULL: rows follow the sequence positions): folded into the
        # attention launch when the append is, else into the append launch, which then also rotates q
        self.rope, self.q_rot = rope, None
        if rope is not None and fused:
            a.rope = ctypes.pointer(rope)
        elif rope is not None:
            self.q_rot = torch.empty_like(q)
            a.q = self.q_rot.data_ptr()
        self.args, self.q = a, q
        self.attn = self.lib.pace_paged_attn_decode if S == 1 else self.lib.pace_paged_attn_verify
        self.stream = nat.current_stream_ptr()
        self.kernel = nat.kernel_name(cache._desc, a)  # the instantiation these arguments launch

    def append(self):
        k, v = self.k, self.v
        if self.rope is not None:
            q, qo = self.q, self.q_rot
            self.nat.check(self.lib.pace_rope_append_paged(
                ctypes.byref(self.cache._desc), ctypes.byref(self.rope), q.data_ptr(), qo.data_ptr(), q.stride(0), q.stride(1),
                q.stride(2), q.shape[1], k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), k.stride(2), self.B, self.T,
                self.table.data_ptr(), self.table.stride(0), self.lens_dev.data_ptr(), -self.T, self.stream))
            return
        self.nat.check(self.lib.pace_kv_append_paged(
            ctypes.byref(self.cache._desc), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), k.stride(2), self.B, self.T,
            self.table.data_ptr(), self.table.stride(0), self.lens_dev.data_ptr(), -self.T, self.stream))

    def gathered(self):
        """Dense K / V ``[B, Hkv, L, D]`` of the cache as a step leaves it (the step's new tokens included)."""
        c = self.cache
        lens, seq_len = c.lens, c.seq_len
        c.lens, c.seq_len = self.lens_after, int(self.lens_after.max())
        try:
            return c.gather(n_rep=1)
        finally:
            c.lens, c.seq_len = lens, seq_len

    def attend(self):
        self.nat.check(self.attn(ctypes.byref(self.cache._desc), ctypes.byref(self.args), self.stream))
        return self.out

    def __call__(self, ev=None):
        if not self.fused:
            self.append()
        if ev:
            ev[0].record()
        self.attend()
        if ev:
            ev[1].record()
