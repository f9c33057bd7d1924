"""Headline benchmark: paged decode attention + KV append, Llama-3-8B shape, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--path api|direct]

A step is one pass of the hot path over one batch: append one new token per
sequence into the block-paged cache, then GQA decode attention over the whole
cache (batch 64, context 4096 -> 4097 tokens read, bf16, block 16, physical
blocks randomly permuted).  Every step runs at the same cache state (the token
lands at position 4096 each time), so bytes per step are constant.  All inputs
are resident in HBM before the timed region.  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import math
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
for _p in (REPO, os.path.join(REPO, "amd-pace_amd")):
    if _p not in sys.path:
        sys.path.insert(0, _p)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published

WORKLOAD = dict(name="llama3-8b-decode", batch=64, context=4096, q_heads=32, kv_heads=8, head_dim=128, block=16)


def algorithmic_bytes(batch, ctx_after, q_heads, kv_heads, head_dim, new_tokens=1):
    """Bytes one step must move: K+V read once at GQA-minimal width, Q read, O written,
    block table and lengths read, new K/V read and written, one slot id per new token."""
    kv_tok = 2 * kv_heads * head_dim * 2
    decode = batch * ctx_after * kv_tok + 2 * batch * q_heads * head_dim * 2 + 4 * batch * math.ceil(ctx_after / 16) + 4 * batch
    append = 2 * (batch * new_tokens * kv_tok) + 4 * batch * new_tokens
    return decode, append


def build_cache(torch, dev, w, seed=1, permute=True):
    """Cache holding `context` tokens per sequence in randomly permuted physical blocks."""
    import numpy as np
    from pace_mi355.llm import PagedKVCache

    B, ctx, hkv, D = w["batch"], w["context"], w["kv_heads"], w["head_dim"]
    per_seq = (ctx + 64 + 15) // 16
    cache = PagedKVCache(ctx + 64, num_kv_heads=hkv, n_rep=w["q_heads"] // hkv, num_blocks=B * per_seq)
    g = torch.Generator(device=dev).manual_seed(seed)
    chunk = 512
    first = True
    for t0 in range(0, ctx, chunk):
        n = min(chunk, ctx - t0)
        k = torch.randn(B, hkv, n, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        v = torch.randn(B, hkv, n, D, generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)
        if first:
            # scramble the free list so that consecutive logical blocks are far apart in HBM
            cache.append_ragged(k[:, :, :1], v[:, :, :1], [0] * B)
            alloc = cache.state.allocator
            ids = alloc.allocate(alloc.num_free)
            if permute:
                np.random.default_rng(seed).shuffle(ids)
            else:
                ids = ids[::-1]
            alloc.free(ids)
            first = False
        cache.update_cache(k, v, 2)
    return cache


def cpu_baseline(torch, w, budget_s=12.0):
    """The reference's CPU path, restated by the oracle, on a bounded sample of the workload:
    BMC cache (its benchmark default) holding GQA-expanded K/V + torch SDPA in bf16."""
    from oracle.attention_ref import lengths_mask_4d, sdpa_native
    from oracle.cache_ref import BMCKVCacheRef, repeat_kv

    cores = torch.get_num_threads()
    B = 8
    ctx, hq, hkv, D = w["context"], w["q_heads"], w["kv_heads"], w["head_dim"]
    n_rep = hq // hkv
    g = torch.Generator().manual_seed(0)
    cache = BMCKVCacheRef(ctx + 128)
    k = torch.randn(B, hkv, ctx, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, hkv, ctx, D, generator=g).to(torch.bfloat16)
    cache.update_cache(repeat_kv(k, n_rep), repeat_kv(v, n_rep), 2)
    del k, v
    k1 = torch.randn(B, hkv, 1, D, generator=g).to(torch.bfloat16)
    v1 = torch.randn(B, hkv, 1, D, generator=g).to(torch.bfloat16)
    q = torch.randn(B, hq, 1, D, generator=g).to(torch.bfloat16)

    def step():
        ke, ve = repeat_kv(k1, n_rep), repeat_kv(v1, n_rep)
        K, V = cache.update_cache(ke, ve, 2)
        n = cache.seq_len
        mask = cache.update_mask(lengths_mask_4d([n] * B, 1, n, torch.bfloat16), n)
        out = sdpa_native(q, K, V, mask)
        cache.remove_cache(1)
        return out

    for _ in range(2):
        step()
    t0 = time.perf_counter()
    n_steps = 0
    while n_steps < 5 or (time.perf_counter() - t0 < budget_s and n_steps < 200):
        step()
        n_steps += 1
    dt = (time.perf_counter() - t0) / n_steps
    decode_b, append_b = algorithmic_bytes(B, ctx + 1, hq, hkv, D)
    return {
        "value": round((decode_b + append_b) / dt / 1e9, 3),
        "unit": "GB/s",
        "tokens_per_s": round(B / dt, 2),
        "ms_per_step": round(dt * 1e3, 3),
        "cores": cores,
        "kind": "port",
        "sample": f"batch {B} of {w['batch']}, context {ctx}, BMC cache with GQA-expanded K/V + torch CPU SDPA bf16; "
                  f"2 warm-up + {n_steps} timed steps; GB/s uses the same GQA-minimal algorithmic bytes as the GPU line",
    }


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--path", choices=("api", "direct"), default="direct",
                    help="direct: C-ABI calls with fixed metadata; api: PagedKVCache.update_cache + MultiHeadAttention")
    ap.add_argument("--partition", type=int, default=0, help="context split size in tokens (0 = library default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-permute", action="store_true", help="keep physical blocks in logical order (diagnostic)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the hot path shards by "
              "sequence with no exchange; see DESIGN.md). Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    from pace_mi355 import _native as nat
    from pace_mi355.ops import MultiHeadAttention

    lib = nat.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    w = WORKLOAD
    B, ctx, hq, hkv, D = w["batch"], w["context"], w["q_heads"], w["kv_heads"], w["head_dim"]
    cache = build_cache(torch, dev, w, permute=not args.no_permute)
    cache.partition_tokens = args.partition
    g = torch.Generator(device=dev).manual_seed(2)
    k1 = torch.randn(B, hkv, 1, D, generator=g, device=dev).to(torch.bfloat16)
    v1 = torch.randn(B, hkv, 1, D, generator=g, device=dev).to(torch.bfloat16)
    q = torch.randn(B, hq, 1, D, generator=g, device=dev).to(torch.bfloat16)
    mha = MultiHeadAttention(dtype=torch.bfloat16)

    if args.path == "api":
        def step(ev=None):
            pk, pv = cache.update_cache(k1, v1, 2)
            if ev:
                ev[0].record()
            out = mha(q, pk, pv)
            if ev:
                ev[1].record()
            cache.remove_cache(1)
            return out
    else:
        # Fixed metadata: lengths after the append, block table, workspace; the new token
        # lands at position `ctx` of every sequence on every step.
        import numpy as np

        lens_after = cache.lens + 1
        cache.state.ensure_capacity(lens_after)
        table = cache.state.device_table()
        lens_dev = torch.from_numpy(lens_after.astype(np.int32)).to(dev)
        out = torch.empty(B, hq, 1, D, dtype=torch.bfloat16, device=dev)
        ws_bytes = int(lib.pace_paged_attn_workspace_bytes(B, hq, 1, D, ctx + 1, args.partition, hkv))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=dev)
        a = nat.PagedAttnArgs()
        a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
        a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
        a.block_table, a.table_stride, a.seq_lens = table.data_ptr(), table.stride(0), lens_dev.data_ptr()
        a.kv_start, a.mask, a.causal = None, None, 1
        a.batch, a.num_q_heads, a.q_len = B, hq, 1
        a.max_seq_len, a.partition_tokens, a.scale = ctx + 1, args.partition, 1.0 / math.sqrt(D)
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws_bytes
        desc = cache._desc
        stream = nat.current_stream_ptr()

        def step(ev=None):
            nat.check(lib.pace_kv_append_paged(ctypes.byref(desc), k1.data_ptr(), v1.data_ptr(), k1.stride(0), k1.stride(1),
                                               k1.stride(2), B, 1, table.data_ptr(), table.stride(0), lens_dev.data_ptr(), -1,
                                               stream))
            if ev:
                ev[0].record()
            nat.check(lib.pace_paged_attn_decode(ctypes.byref(desc), ctypes.byref(a), stream))
            if ev:
                ev[1].record()
            return out

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for i in range(args.steps):
        step(events[i])
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    attn_ms = sum(e0.elapsed_time(e1) for e0, e1 in events) / args.steps

    decode_b, append_b = algorithmic_bytes(B, ctx + 1, hq, hkv, D)
    step_bytes = decode_b + append_b
    ms_per_step = dt * 1e3 / args.steps
    gbs = step_bytes / (dt / args.steps) / 1e9
    achieved = decode_b / (attn_ms * 1e-3) / 1e9
    line = {
        "metric": "decode-attention+KV-append HBM GB/s (% of peak) & tokens/s, 8B shape, 1 GPU",
        "value": round(gbs, 1),
        "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "tokens_per_s": round(B * args.steps / dt, 1),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "Llama-3-8B-shape single-layer decode: batch 64, context 4096 (+1 appended), 32 Q / 8 KV heads, "
                        "head_dim 128, KV block 16, seeded random physical block permutation, 1-token append + GQA decode",
            "bytes_per_step": step_bytes,
            "path": args.path,
            "partition_tokens": args.partition,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "paged_attn_kernel<128,1,false> (+ merge)",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": None,
            "bytes_per_launch": decode_b,
            "avg_launch_ms": round(attn_ms, 5),
        },
    }
    if not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(torch, w)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
