"""GPU parity at the benchmark configurations.  Small ones are compared in full with the CPU
oracle; the large ones through sampled sequences (oracle) plus size-independent properties
(gather == source, invariance under block permutation / compaction, truncate == prefix)."""
import math

import numpy as np
import pytest
import torch

from helpers import assert_attention_close
from oracle.attention_ref import lengths_mask_4d, sdpa_fp32
from oracle.cache_ref import DynamicKVCacheRef, repeat_kv

pytestmark = pytest.mark.gpu


def _randn_bf16(shape, gen, dev):
    return torch.randn(*shape, generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)


def _scramble(cache, k1, v1, seed, history=False):
    """Initialise the cache's state and leave its free list in a seeded, fragmented order: a shuffle, or what a
    seeded admit / retire history of sequences leaves behind (the ragged serving mix)."""
    cache.append_ragged(k1, v1, [0] * k1.shape[0])
    alloc = cache.state.allocator
    if history:
        from pace_mi355.utils.history import alloc_free_history

        alloc_free_history(alloc, seed, 8, 1024)
        return
    ids = alloc.allocate(alloc.num_free)
    np.random.default_rng(seed).shuffle(ids)
    alloc.free(ids)


def _fill(cache, lens, gen, dev, hkv, D, chunk=1024, seed=0, history=False):
    """Append lens[b] tokens to each sequence; returns the source K/V as [B, hkv, max, D] on the GPU."""
    B, T = len(lens), max(lens)
    K = torch.zeros(B, hkv, T, D, dtype=torch.bfloat16, device=dev)
    V = torch.zeros_like(K)
    lens = np.asarray(lens)
    first = True
    for t0 in range(0, T, chunk):
        n = min(chunk, T - t0)
        k, v = _randn_bf16((B, hkv, n, D), gen, dev), _randn_bf16((B, hkv, n, D), gen, dev)
        if first:
            _scramble(cache, k[:, :, :1], v[:, :, :1], seed, history)
            first = False
        counts = np.clip(lens - t0, 0, n)
        cache.append_ragged(k, v, counts)
        K[:, :, t0 : t0 + n], V[:, :, t0 : t0 + n] = k, v
    for b, n in enumerate(lens):  # rows past each length were never appended
        K[b, :, n:], V[b, :, n:] = 0, 0
    return K, V


def _oracle_rows(q, K, V, lens, rows, n_rep):
    """fp32 oracle attention for the sampled batch rows."""
    idx = torch.tensor(rows)
    qs, Ks, Vs = q[idx].cpu(), K[idx].cpu(), V[idx].cpu()
    ls = [int(lens[r]) for r in rows]
    L = max(ls)
    mask = lengths_mask_4d(ls, q.shape[2], L, torch.float32)
    return sdpa_fp32(qs, repeat_kv(Ks[:, :, :L], n_rep), repeat_kv(Vs[:, :, :L], n_rep), mask)


def test_cfg1_plumbing_two_layers_full_parity(device):
    """2 layers, B=4, contexts U[64,512] (seed 0), 32 Q / 8 KV heads, D=128: every step appends one
    token per sequence and decodes; cache contents bit-exact, attention within tolerance."""
    from pace_mi355.llm import KVCacheManager, KVCacheType
    from pace_mi355.ops import MultiHeadAttention

    class Cfg:
        num_hidden_layers, num_attention_heads, num_key_value_heads = 2, 32, 8

    torch.manual_seed(0)
    B, Hq, Hkv, D = 4, 32, 8, 128
    lens = torch.randint(64, 513, (B,)).tolist()
    T = max(lens)
    mgr = KVCacheManager(Cfg(), T + 8, KVCacheType.PAGED)
    mha = MultiHeadAttention(dtype=torch.bfloat16)
    refs = [DynamicKVCacheRef(T + 8) for _ in range(2)]
    # left-padded prompt as the reference batches it: shared length T, per-sequence pad T - len
    pad = [T - n for n in lens]
    mask2d = torch.ones(B, T, dtype=torch.long)
    for b, p in enumerate(pad):
        mask2d[b, :p] = 0
    from oracle.attention_ref import causal_mask_4d

    for layer in range(2):
        k, v = torch.randn(B, Hkv, T, D).bfloat16(), torch.randn(B, Hkv, T, D).bfloat16()
        refs[layer].update_cache(repeat_kv(k, 4), repeat_kv(v, 4), 2)
        mgr[layer].update_cache(repeat_kv(k, 4).to(device), repeat_kv(v, 4).to(device), 2)
    for step in range(3):
        mask2d = torch.cat([mask2d, torch.ones(B, 1, dtype=torch.long)], 1)
        L = mask2d.shape[1]
        m4 = causal_mask_4d(mask2d, 1, L, torch.bfloat16)
        for layer in range(2):
            k, v, q = torch.randn(B, Hkv, 1, D).bfloat16(), torch.randn(B, Hkv, 1, D).bfloat16(), torch.randn(B, Hq, 1, D).bfloat16()
            rk, rv = refs[layer].update_cache(repeat_kv(k, 4), repeat_kv(v, 4), 2)
            pk, pv = mgr[layer].update_cache(repeat_kv(k, 4).to(device), repeat_kv(v, 4).to(device), 2)
            assert torch.equal(pk.dense().cpu(), rk) and torch.equal(pv.dense().cpu(), rv)
            out = mha(q.to(device), pk, pv, attention_mask=mgr.update_mask(m4.to(device), L))
            assert_attention_close(out, sdpa_fp32(q, rk, rv, m4), f"step {step} layer {layer}")
        assert len(mgr) == L


def test_cfg2_headline_shape_properties(device):
    """B=64, ctx 4096 (+1), 32 Q / 8 KV heads, permuted physical blocks."""
    from pace_mi355.llm import PagedKVCache

    B, Hq, Hkv, D, ctx = 64, 32, 8, 128, 4096
    gen = torch.Generator(device=device).manual_seed(1)
    cache = PagedKVCache(ctx + 64, num_kv_heads=Hkv, n_rep=4, num_blocks=B * 260)
    K, V = _fill(cache, [ctx] * B, gen, device, Hkv, D, seed=1)
    k1, v1 = _randn_bf16((B, Hkv, 1, D), gen, device), _randn_bf16((B, Hkv, 1, D), gen, device)
    q = _randn_bf16((B, Hq, 1, D), gen, device)
    cache.update_cache(k1, v1, 2)
    K, V = torch.cat([K, k1], 2), torch.cat([V, v1], 2)
    gk, gv = cache.gather(n_rep=1)
    assert torch.equal(gk, K) and torch.equal(gv, V), "gather must reproduce the appended stream bit for bit"
    out = cache.attend(q)
    rows = [0, 17, 63]
    assert_attention_close(out[rows], _oracle_rows(q, K, V, [ctx + 1] * B, rows, 4), "cfg2 sampled rows")
    # same logical cache in sequential physical order -> identical bits
    seq = PagedKVCache(ctx + 64, num_kv_heads=Hkv, n_rep=4, num_blocks=B * 260)
    seq.update_cache(K, V, 2)
    assert not np.array_equal(seq.state.table, cache.state.table)
    assert torch.equal(seq.attend(q), out)
    # explicit partitions + merge kernel agree with the single-pass result
    cache.partition_tokens = 1024
    assert_attention_close(cache.attend(q), out.float(), "partitioned vs single pass")


def test_cfg3_ragged_mix_properties(device):
    """B=256, contexts log-uniform in [128, 16384] (seed 2), pool 1.3x live tokens, fragmented free list."""
    from pace_mi355.llm import PagedKVCache

    B, Hq, Hkv, D = 256, 32, 8, 128
    rng = np.random.default_rng(2)
    lens = np.round(np.exp(rng.uniform(math.log(128), math.log(16384), B))).astype(int).tolist()
    live_blocks = sum((n + 15) // 16 for n in lens)
    cache = PagedKVCache(max(lens) + 16, num_kv_heads=Hkv, n_rep=4, num_blocks=int(1.3 * live_blocks))
    gen = torch.Generator(device=device).manual_seed(3)
    K, V = _fill(cache, lens, gen, device, Hkv, D, chunk=2048, seed=3, history=True)
    # append one more token everywhere, then decode
    k1, v1 = _randn_bf16((B, Hkv, 1, D), gen, device), _randn_bf16((B, Hkv, 1, D), gen, device)
    cache.update_cache(k1, v1, 2)
    K = torch.cat([K, torch.zeros_like(k1)], 2)
    V = torch.cat([V, torch.zeros_like(v1)], 2)
    for b, n in enumerate(lens):
        K[b, :, n], V[b, :, n] = k1[b, :, 0], v1[b, :, 0]
    lens1 = [n + 1 for n in lens]
    gk, gv = cache.gather(n_rep=1)
    assert torch.equal(gk, K) and torch.equal(gv, V)
    q = _randn_bf16((B, Hq, 1, D), gen, device)
    out = cache.attend(q)
    order = np.argsort(lens)
    rows = [int(order[0]), int(order[B // 2]), int(order[-1]), 5]
    assert_attention_close(out[rows], _oracle_rows(q, K, V, lens1, rows, 4), "cfg3 sampled rows")
    moved = cache.compact()
    assert moved <= live_blocks + B
    assert torch.equal(cache.attend(q), out), "compaction must not change attention output"
    gk2, _ = cache.gather(n_rep=1)
    assert torch.equal(gk2, K)


def test_cfg4_pard_verify_and_rollback(device):
    """B=32, contexts U[1024,8192] (seed 4), 8 draft tokens appended, causal 8-query attention,
    then a seeded 0..8 rollback per sequence (seed 5)."""
    from pace_mi355.llm import PagedKVCache

    B, Hq, Hkv, D, S = 32, 32, 8, 128, 8
    lens = np.random.default_rng(4).integers(1024, 8193, B).tolist()
    cache = PagedKVCache(max(lens) + 64, num_kv_heads=Hkv, n_rep=4, num_blocks=B * ((max(lens) + 64) // 16 + 1))
    gen = torch.Generator(device=device).manual_seed(4)
    K, V = _fill(cache, lens, gen, device, Hkv, D, chunk=2048, seed=4)
    kd, vd = _randn_bf16((B, Hkv, S, D), gen, device), _randn_bf16((B, Hkv, S, D), gen, device)
    cache.update_cache(kd, vd, 2)
    K = torch.cat([K, torch.zeros_like(kd)], 2)
    V = torch.cat([V, torch.zeros_like(vd)], 2)
    for b, n in enumerate(lens):
        K[b, :, n : n + S], V[b, :, n : n + S] = kd[b], vd[b]
    lens_v = [n + S for n in lens]
    q = _randn_bf16((B, Hq, S, D), gen, device)
    out = cache.attend(q)
    rows = [0, int(np.argmax(lens)), int(np.argmin(lens))]
    assert_attention_close(out[rows], _oracle_rows(q, K, V, lens_v, rows, 4), "cfg4 verify rows")
    free_before = cache.state.allocator.num_free
    rej = np.random.default_rng(5).integers(0, 9, B)
    cache.truncate(rej)
    lens_r = [n - int(r) for n, r in zip(lens_v, rej)]
    assert cache.lens.tolist() == lens_r
    freed = sum((a + 15) // 16 - (c + 15) // 16 for a, c in zip(lens_v, lens_r))
    assert cache.state.allocator.num_free == free_before + freed
    gk, gv = cache.gather(n_rep=1)
    for b in (0, 7, 31):
        assert torch.equal(gk[b, :, : lens_r[b]], K[b, :, : lens_r[b]]) and torch.count_nonzero(gk[b, :, lens_r[b] :]) == 0
        assert torch.equal(gv[b, :, : lens_r[b]], V[b, :, : lens_r[b]])
    # the next decode step reads exactly the accepted prefix
    q1 = q[:, :, :1].contiguous()
    out1 = cache.attend(q1)
    assert_attention_close(out1[rows], _oracle_rows(q1, K, V, lens_r, rows, 4), "decode after rollback")


def test_cfg5_evict_compact_decode_70b_shape(device):
    """64 Q / 8 KV heads, B=8, ctx 32768: evict a seeded 40% of blocks (seed 6), compact, decode."""
    from pace_mi355.llm import PagedKVCache

    B, Hq, Hkv, D, ctx = 8, 64, 8, 128, 32768
    cache = PagedKVCache(ctx, num_kv_heads=Hkv, n_rep=8, num_blocks=B * ctx // 16)
    gen = torch.Generator(device=device).manual_seed(6)
    K, V = _fill(cache, [ctx] * B, gen, device, Hkv, D, chunk=4096, seed=6)
    rng = np.random.default_rng(6)
    keep_rows = []
    for b in range(B):
        drop = np.sort(rng.choice(ctx // 16, size=int(0.4 * ctx // 16), replace=False))
        cache.evict_blocks(b, drop.tolist())
        keep = np.ones(ctx // 16, dtype=bool)
        keep[drop] = False
        keep_rows.append(torch.from_numpy(np.repeat(keep, 16)).to(device))
    n_live = cache.state.live_block_count()
    assert n_live == B * (ctx // 16 - int(0.4 * ctx // 16))
    Ks = torch.stack([K[b][:, keep_rows[b]] for b in range(B)])  # surviving tokens, in order
    Vs = torch.stack([V[b][:, keep_rows[b]] for b in range(B)])
    q = _randn_bf16((B, Hq, 1, D), gen, device)
    before = cache.attend(q)
    moved = cache.compact()
    assert 0 < moved <= n_live
    used = np.concatenate([cache.state.table[b, : cache.state.n_blocks[b]] for b in range(B)])
    assert sorted(used.tolist()) == list(range(n_live))
    gk, gv = cache.gather(n_rep=1)
    assert torch.equal(gk, Ks) and torch.equal(gv, Vs), "compacted cache == cache built from the survivors only"
    after = cache.attend(q)
    assert torch.equal(before, after)
    rows = [0, 7]
    assert_attention_close(after[rows], _oracle_rows(q, Ks, Vs, cache.lens.tolist(), rows, 8), "cfg5 decode")


def _oracle_all_rows(q, K, V, lens, n_rep, out, what, chunk=8):
    """Every sequence of the batch against the fp32 oracle, `chunk` sequences at a time."""
    for b0 in range(0, q.shape[0], chunk):
        rows = list(range(b0, min(b0 + chunk, q.shape[0])))
        assert_attention_close(out[rows], _oracle_rows(q, K, V, lens, rows, n_rep), f"{what}, sequences {rows[0]}..{rows[-1]}")


def test_cfg2_headline_launch_as_benchmarked(device):
    """The launch the headline figure is timed on, as bench.py issues it: the fused append + decode kernel started
    through the C ABI with frozen metadata and a work list, batch 64 x 4096 (+1), permuted pool.  All 64 sequences
    are compared with the fp32 oracle, and the slot the launch writes (position 4096) bit for bit."""
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.utils.fixed_step import FixedStep

    B, Hq, Hkv, D, ctx = 64, 32, 8, 128, 4096
    gen = torch.Generator(device=device).manual_seed(1)
    cache = PagedKVCache(ctx + 64, num_kv_heads=Hkv, n_rep=4, num_blocks=B * 260)
    K, V = _fill(cache, [ctx] * B, gen, device, Hkv, D, seed=1)
    k1, v1 = _randn_bf16((B, Hkv, 1, D), gen, device), _randn_bf16((B, Hkv, 1, D), gen, device)
    q = _randn_bf16((B, Hq, 1, D), gen, device)
    step = FixedStep(torch, cache, q, k1, v1, fused=True)
    assert step.kernel == "pace_kv::paged_attn_kernel<128, 1, false, 4, 2, 8, true, false, true>", step.kernel
    assert step.n_items >= B and step.args.work_items, "the benchmarked launch runs from a work list"
    pool_before = cache.pool.clone()
    step()  # one fused launch: stores token 4096 of every sequence and attends over 4097 tokens
    torch.cuda.synchronize()
    out = step.out.clone()
    K1, V1 = torch.cat([K, k1], 2), torch.cat([V, v1], 2)
    _oracle_all_rows(q, K1, V1, [ctx + 1] * B, 4, out, "cfg2 fused launch")
    # what the launch stored: the new token's slot holds k1 / v1 bit for bit, nothing else in the pool changed
    cache.lens = cache.lens + 1  # (the direct call does not move the host-side lengths)
    cache.seq_len += 1
    gk, gv = cache.gather(n_rep=1)
    assert torch.equal(gk[:, :, ctx], k1[:, :, 0]) and torch.equal(gv[:, :, ctx], v1[:, :, 0]), "slot 4096 must hold the new token"
    assert torch.equal(gk, K1) and torch.equal(gv, V1)
    changed = (cache.pool != pool_before).flatten(1).any(1).sum().item()
    assert changed <= B, f"the launch rewrote {changed} blocks; it may touch one per sequence"
    # a second launch on the same state (what the timed loop does) gives the same bits
    step()
    torch.cuda.synchronize()
    assert torch.equal(step.out, out)


def test_cfg4_fused_verify_launch_as_benchmarked(device):
    """The cfg4 launch of bench.py --workload verify: 8 draft tokens per sequence appended by the attention launch
    itself (fused), causal 8-query attention, batch 32 with contexts U[1024, 8192]; every sequence against the
    oracle, the eight new slots of every sequence bit for bit."""
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.utils.fixed_step import FixedStep

    B, Hq, Hkv, D, S = 32, 32, 8, 128, 8
    lens = np.random.default_rng(4).integers(1024, 8193, B).tolist()
    cache = PagedKVCache(max(lens) + 64, num_kv_heads=Hkv, n_rep=4, num_blocks=B * ((max(lens) + 64) // 16 + 1))
    gen = torch.Generator(device=device).manual_seed(4)
    K, V = _fill(cache, lens, gen, device, Hkv, D, chunk=2048, seed=4)
    kd, vd = _randn_bf16((B, Hkv, S, D), gen, device), _randn_bf16((B, Hkv, S, D), gen, device)
    q = _randn_bf16((B, Hq, S, D), gen, device)
    step = FixedStep(torch, cache, q, kd, vd, fused=True)
    assert "paged_attn_kernel<128, 2, false" in step.kernel and ", true, false, true>" in step.kernel, step.kernel
    step()
    torch.cuda.synchronize()
    out = step.out.clone()
    K1 = torch.cat([K, torch.zeros_like(kd)], 2)
    V1 = torch.cat([V, torch.zeros_like(vd)], 2)
    for b, n in enumerate(lens):
        K1[b, :, n : n + S], V1[b, :, n : n + S] = kd[b], vd[b]
    lens_v = [n + S for n in lens]
    _oracle_all_rows(q, K1, V1, lens_v, 4, out, "cfg4 fused verify launch")
    cache.lens = cache.lens + S
    cache.seq_len = int(cache.lens.max())
    gk, gv = cache.gather(n_rep=1)
    assert torch.equal(gk, K1) and torch.equal(gv, V1), "the eight new slots of every sequence hold the drafts bit for bit"
    step()
    torch.cuda.synchronize()
    assert torch.equal(step.out, out)
