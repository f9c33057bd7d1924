"""Benchmarks of the KV-cache hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload decode-8b]

The default workload is the headline one: Llama-3-8B-shape single-layer decode, batch 64,
context 4096, bf16, 32 Q / 8 KV heads, head_dim 128, KV block 16, physical blocks randomly
permuted.  A step is one pass of the hot path over one batch: append one new token per
sequence into the block-paged cache, then GQA decode attention over the whole cache.
Every step runs at the same cache state (the token lands at position 4096 each time), so
the bytes per step are constant; the steps rotate over --layers distinct pools (default 4) so that
every step reads its K / V from HBM, not from what the step before left in the last-level cache.  All inputs are resident in HBM before the timed region.
One JSON line is printed.

Other workloads (same JSON shape, `config.workload` names them):
  ragged    batch 256, contexts log-uniform in [128, 16384], pool 1.3x live tokens:
            append + decode per step; gather timed beside it
  verify    batch 32, contexts U[1024, 8192], 8 draft tokens appended + causal 8-query attention
  prefill / dense-prefill   a 512-token chunk over 3584 cached tokens through the paged path; the dense
            op on 2048 x 2048 with the additive causal mask (roofline against the matrix-core peak)
  decode-gptj   the headline step at GPT-J-6B's attention shape (16 heads of 256, batch 64 x 2048)
  dense-f32     the dense op on fp32 tensors (the general kernel; roofline against the fp32 matrix-core peak)
  decode-f32pool   the headline step over a pool of fp32 rows (an fp32 model on the paged cache)
  compact   Llama-3-70B-shape KV, batch 8, context 32768: evict 40% of the blocks, then time the
            compaction copy and the decode over the compacted cache
  gather / append    the block-table gather (dense and packed output) and the stand-alone append (1 / 8 / 512
            tokens per sequence) at the headline shape, each against the HBM roofline
  copy-calibration   block copy of a known byte count, used to scale the HBM byte counters
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
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16 matrix-core peak, published
MFMA_F32_PEAK_TFLOPS = 157.3  # MI355X fp32 matrix-core peak, published
METRIC = "decode-attention+KV-append HBM GB/s (% of peak) & tokens/s, 8B shape, 1 GPU"



def measured_traffic(kernel):
    """HBM bytes per launch of `kernel` as the committed counter summary states them, or None.

    profiles/decode_8b_paged_attn_kernel.txt (rocprofv3 FETCH_SIZE / WRITE_SIZE runs of the default workload,
    scaled by the same counters on the copy-calibration workload) ends in a line
    `traffic_bytes_per_launch <bytes> kernel <name as the profiler prints it>`.  The figure is used only when
    that name is the instantiation this run launches (asked from the library), so a change of the kernel's
    template arguments drops the figure instead of carrying a stale one."""
    path = os.path.join(REPO, "profiles", "decode_8b_paged_attn_kernel.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch "):
                _, nbytes, _, name = line.rstrip("\n").split(" ", 3)
                if name.strip() == kernel:
                    return int(nbytes)
    except OSError:
        pass
    return None


def kv_token_bytes(kv_heads, head_dim):
    return 2 * kv_heads * head_dim * 2  # K and V, bf16


def decode_bytes(lens, q_heads, kv_heads, head_dim, q_len=1):
    """Algorithmic bytes of one attention launch: K+V read once at GQA-minimal width, Q read,
    O written, block table and lengths read."""
    B = len(lens)
    return (sum(lens) * kv_token_bytes(kv_heads, head_dim) + 2 * B * q_heads * q_len * head_dim * 2
            + 4 * sum(math.ceil(n / 16) for n in lens) + 4 * B)


def append_bytes(batch, new_tokens, kv_heads, head_dim):
    """New K/V read and written, one slot id per new token."""
    return 2 * batch * new_tokens * kv_token_bytes(kv_heads, head_dim) + 4 * batch * new_tokens


from pace_mi355.utils.fixed_step import FixedStep, build_cache, randn_bf16 as _randn_bf16  # noqa: E402


EVENT_EVERY = 8  # an event record costs several microseconds of GPU timeline; bracket one launch in eight


def run_timed(torch, step, steps, warmup):
    """W untimed steps, then exactly K timed steps bracketed by synchronize.  Inside the timed region
    the attention launch of every eighth step is bracketed by HIP events on the launch stream.
    Returns (s per step, ms per launch)."""
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
              for _ in range((steps + EVENT_EVERY - 1) // EVENT_EVERY)]
    t0 = time.perf_counter()
    for i in range(steps):
        step(events[i // EVENT_EVERY] if i % EVENT_EVERY == 0 else None)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    return dt, sum(a.elapsed_time(b) for a, b in events) / len(events)


def time_call(torch, fn, reps=20, warmup=3):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for a, b in ev:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return sum(a.elapsed_time(b) for a, b in ev) / reps


def roofline(kernel, nbytes, ms, extra=None):
    gbs = nbytes / (ms * 1e-3) / 1e9
    d = {"bound": "hbm", "kernel": kernel, "achieved": round(gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
         "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": None, "bytes_per_launch": int(nbytes), "avg_launch_ms": round(ms, 5)}
    if extra:
        d.update(extra)
    return d


def result_line(args, workload, step_bytes, tokens_per_step, dt, roof, extra_cfg=None, extra=None):
    gbs = step_bytes / dt / 1e9
    line = {
        "metric": METRIC,
        "value": round(gbs, 1),
        "unit": "GB/s",
        "pct_of_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "tokens_per_s": round(tokens_per_step / dt, 1),
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": workload, "bytes_per_step": int(step_bytes), "partition_tokens": args.partition},
        "roofline": roof,
    }
    if extra_cfg:
        line["config"].update(extra_cfg)
    if extra:
        line.update(extra)
    return line


CHECK_NOTE = ("last timed step vs the fp32 CPU oracle (caps 2e-2 max abs / 1e-2 relative per sequence); slots of the new "
              "tokens bit-exact for every sequence")


def check_attention(torch, q, out, gk, gv, lens, rows):
    """Output rows of the sampled sequences `rows` against the fp32 oracle (the restated reference attention on the
    CPU) over the dense K / V `gk`, `gv` [B, Hkv, L, D] gathered back from the pool.  Caps: max abs error 2e-2,
    relative error (per sequence, Euclidean norm) 1e-2."""
    from oracle.attention_ref import lengths_mask_4d, sdpa_fp32
    from oracle.cache_ref import repeat_kv

    S, n_rep = q.shape[2], q.shape[1] // gk.shape[1]
    idx = torch.tensor(rows, device=gk.device)
    ls = [int(lens[r]) for r in rows]
    L = max(ls)
    got = out[idx].float().cpu()
    ref = sdpa_fp32(q[idx].cpu(), repeat_kv(gk[idx][:, :, :L].cpu(), n_rep), repeat_kv(gv[idx][:, :, :L].cpu(), n_rep),
                    lengths_mask_4d(ls, S, L, torch.float32))
    err = (got - ref).abs()
    rel = float((err.flatten(1).norm(dim=1) / ref.flatten(1).norm(dim=1)).max())
    max_abs = float(err.max())
    ok = bool(max_abs <= 2e-2 and rel <= 1e-2 and not torch.isnan(got).any())
    return {"checked": ok, "max_abs_err": round(max_abs, 6), "max_rel_err": round(rel, 6), "checked_sequences": [int(r) for r in rows]}


def self_check(torch, step, rows):
    """After the timed region: the last step's output for the sampled sequences against the oracle, and the slots
    the step's new tokens were stored in against the tokens themselves, bit for bit, for every sequence."""
    torch.cuda.synchronize()
    gk, gv = step.gathered()
    T = step.T
    slots_ok = True
    for b, n in enumerate(step.lens_after.tolist()):
        slots_ok = slots_ok and torch.equal(gk[b, :, n - T:n], step.k[b]) and torch.equal(gv[b, :, n - T:n], step.v[b])
    res = check_attention(torch, step.q, step.out, gk, gv, step.lens_after, rows)
    res["appended_slots_bit_exact"] = bool(slots_ok)
    res["checked"] = bool(res["checked"] and slots_ok)
    res["check"] = CHECK_NOTE
    return res


def spread_rows(lens):
    """Sequences to sample: the shortest, the median, the longest and the last of the batch."""
    import numpy as np

    order = np.argsort(np.asarray(lens), kind="stable")
    return sorted({int(order[0]), int(order[len(order) // 2]), int(order[-1]), len(lens) - 1})


# ---- workloads ---------------------------------------------------------------------------------
def wl_decode_8b(torch, dev, args):
    return _wl_decode(torch, dev, args, (64, 4096, 32, 8, 128),
                      "Llama-3-8B-shape single-layer decode: batch 64, context 4096 (+1 appended), 32 Q / 8 KV heads, head_dim 128, "
                      "KV block 16, seeded random physical block permutation, 1-token append + GQA decode",
                      True, with_cpu=True)


def wl_decode_gptj(torch, dev, args):
    """The same step at GPT-J-6B's attention shape (16 heads of 256, no GQA): the same bytes per step
    as the headline with half the context."""
    return _wl_decode(torch, dev, args, (64, 2048, 16, 16, 256),
                      "GPT-J-6B-shape single-layer decode: batch 64, context 2048 (+1 appended), 16 Q / 16 KV heads, head_dim 256, "
                      "KV block 16, seeded random physical block permutation, 1-token append + decode", False, with_cpu=False)


def _wl_decode(torch, dev, args, shape, label, has_traffic_profile, with_cpu):
    B, ctx, hq, hkv, D = shape
    if args.batch or args.context:
        B, ctx = args.batch or B, args.context or ctx
        label = f"{label} -- with batch {B} and context {ctx} instead"
    # One pool per layer, each with its own seeded block permutation: step i runs on pool i mod N, as a
    # decoder walks its layers (pace/llm/models/llama.py:312-315), so no step finds the K / V of the step
    # before it in the 256 MB last-level cache.
    n_layers = max(1, args.layers)
    caches = [build_cache(torch, dev, [ctx] * B, hq, hkv, D, seed=1 + 100 * i, permute=not args.no_permute,
                          headroom=64 + args.steps + args.warmup) for i in range(n_layers)]
    cache = caches[0]
    for c in caches:
        c.partition_tokens = args.partition
    g = torch.Generator(device=dev).manual_seed(2)
    k1, v1 = _randn_bf16(torch, (B, hkv, 1, D), g, dev), _randn_bf16(torch, (B, hkv, 1, D), g, dev)
    q = _randn_bf16(torch, (B, hq, 1, D), g, dev)
    keep = []
    turn = [0]
    if args.path == "api":
        from pace_mi355.ops import MultiHeadAttention

        mha = MultiHeadAttention(dtype=torch.bfloat16)
        # --mask: the call exactly as the reference's models make it (llama.py:151-165): K/V arrive
        # expanded by repeat_kv, and the additive [B,1,1,L] mask of the step is passed along
        n_rep = hq // hkv
        ka, va = (k1.repeat_interleave(n_rep, dim=1), v1.repeat_interleave(n_rep, dim=1)) if args.mask else (k1, v1)
        mask_all = torch.zeros(B, 1, 1, ctx + 64 + args.steps + args.warmup, device=dev, dtype=torch.bfloat16)
        keep.extend([ka, va, mask_all])

        def step(ev=None):
            c = caches[turn[0] % n_layers]
            turn[0] += 1
            pk, pv = c.update_cache(ka, va, 2)  # the context of a layer grows by one token per step on this path
            if ev:
                ev[0].record()
            mha(q, pk, pv, attention_mask=mask_all[..., : c.seq_len] if args.mask else None)
            if ev:
                ev[1].record()
    elif args.path == "graph":
        from pace_mi355.llm.graph import DecodeGraph
        from pace_mi355.ops import MultiHeadAttention

        # the same calls as --path api, captured once per layer pool into a HIP graph and replayed per step
        mha = MultiHeadAttention(dtype=torch.bfloat16)
        outs = {}

        def one(c):
            def fn():
                pk, pv = c.update_cache(k1, v1, 2)
                return mha(q, pk, pv)
            return fn
        graphs = [DecodeGraph([c], one(c), -(-(args.steps + args.warmup) // n_layers) + 1) for c in caches]
        keep.append(graphs)

        def step(ev=None):
            gr = graphs[turn[0] % n_layers]
            turn[0] += 1
            if ev:
                ev[0].record()
            gr.replay()
            if ev:
                ev[1].record()
    else:
        rope = None
        if args.rope:  # q and k arrive un-rotated; llama-3 tables as RotaryEmbedding builds them
            from pace_mi355 import _native as nat
            from pace_mi355.ops import RotaryEmbedding

            mod = RotaryEmbedding(dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                       original_max_position_embeddings=8192), D, 8192, 500000.0)
            cos, sin = mod.device_tables(dev)
            keep.extend([cos, sin])
            rope = nat.RopeDesc(cos=cos.data_ptr(), sin=sin.data_ptr(), table_dtype=nat.DTYPE_BF16, table_rows=cos.shape[0],
                                rotary_dim=D, interleaved=0, positions=None, pos_stride_b=0)
        fixed = [FixedStep(torch, c, q, k1, v1, args.partition, fused=not args.no_fuse, rope=rope) for c in caches]

        def step(ev=None):
            f = fixed[turn[0] % n_layers]
            turn[0] += 1
            f(ev)
    dt, attn_ms = run_timed(torch, step, args.steps, args.warmup)
    if args.path in ("api", "graph"):  # average context over the timed steps (each layer's cache grows once every n_layers steps)
        ctx = ctx + (args.warmup + (args.steps - 1) // 2) // n_layers
    dec = decode_bytes([ctx + 1] * B, hq, hkv, D)
    fused = args.path == "direct" and not args.no_fuse or args.path in ("api", "graph")
    launch_bytes = dec + (append_bytes(B, 1, hkv, D) if fused else 0)
    kernel = fixed[0].kernel if args.path == "direct" else "pace_kv::paged_attn_kernel (through PagedKVCache / MultiHeadAttention)"
    traffic = measured_traffic(kernel) if has_traffic_profile else None
    check = None
    if args.path == "direct" and not args.rope and not args.no_check:
        check = self_check(torch, fixed[(turn[0] - 1) % n_layers], spread_rows([ctx] * B))
    line = result_line(
        args, label, dec + append_bytes(B, 1, hkv, D), B, dt,
        roofline(kernel + (" (decode, append fused in)" if fused else " (decode)"), launch_bytes, attn_ms, {"traffic": traffic}),
        {"path": args.path, "append_fused": fused, "rope": bool(args.rope and args.path == "direct"),
         "mask": bool(args.mask and args.path == "api"), "layers": n_layers,
         "distinct_pool_bytes": int(n_layers * B * ctx * kv_token_bytes(hkv, D))}, extra=check)
    if with_cpu and not args.no_cpu_baseline:
        line["cpu_baseline"] = cpu_baseline(torch, B, ctx, hq, hkv, D)
    return line


def wl_ragged(torch, dev, args):
    import numpy as np

    B, hq, hkv, D = 256, 32, 8, 128
    rng = np.random.default_rng(2)
    lens = np.round(np.exp(rng.uniform(math.log(128), math.log(16384), B))).astype(int).tolist()
    # pool 1.3x the live blocks, free list as a seeded admit / retire history of sequences leaves it (seed 3)
    cache = build_cache(torch, dev, lens, hq, hkv, D, seed=3, pool_factor=1.3, headroom=16, history=True)
    cache.partition_tokens = args.partition
    g = torch.Generator(device=dev).manual_seed(4)
    k1, v1 = _randn_bf16(torch, (B, hkv, 1, D), g, dev), _randn_bf16(torch, (B, hkv, 1, D), g, dev)
    q = _randn_bf16(torch, (B, hq, 1, D), g, dev)
    step = FixedStep(torch, cache, q, k1, v1, args.partition, fused=not args.no_fuse)
    dt, attn_ms = run_timed(torch, step, args.steps, args.warmup)
    lens1 = [n + 1 for n in lens]
    dec = decode_bytes(lens1, hq, hkv, D)
    gather_b = 2 * sum(lens) * kv_token_bytes(hkv, D)
    forms = {}
    for form in ("packed", "dense", "dense_zero_fill"):
        fn = gather_call(torch, cache, form)
        forms[form] = roofline(f"kv_gather_kernel<128,{'false' if form == 'dense_zero_fill' else 'true'}> ({form.replace('_', ' ')})", gather_b,
                               time_call(torch, fn, reps=5, warmup=1))
    check = {} if args.no_check else self_check(torch, step, spread_rows(lens1))
    return result_line(
        args, f"ragged serving mix: batch 256, contexts log-uniform [128,16384] (seed 2, {sum(lens)} live tokens), pool 1.3x "
        "with the free list left by a seeded admit / retire history (seed 3), "
        "1-token append + GQA decode", dec + append_bytes(B, 1, hkv, D), B, dt,
        roofline(step.kernel + " (decode, ragged) + merge", dec, attn_ms, {"work_items": step.n_items, "max_parts": step.max_parts}),
        extra=dict(check, gather=forms))


def gather_call(torch, cache, form):
    """A closure that runs one gather of the whole cache into preallocated outputs (KV heads only, no
    repeat_kv expansion).  form: "packed" ([sum len][H][D] + cu_seqlens), "dense" ([B][H][Lmax][D], rows past
    each length left alone) or "dense_zero_fill" (the same with the padding written as zeros)."""
    import numpy as np
    from pace_mi355 import _native as nat

    lib, dev = nat.load(), cache.pool.device
    st = cache.state
    table, (lens_dev, bias) = st.device_table(), st.device_lens(cache.lens)
    B, H, D, L = cache.batch, cache.num_kv_heads, cache.head_dim, int(cache.lens.max())
    if form == "packed":
        cu = np.zeros(B + 1, dtype=np.int64)
        np.cumsum(cache.lens, out=cu[1:])
        cu_dev = torch.from_numpy(cu.astype(np.int32)).to(dev)
        k, v = (torch.empty(int(cu[-1]), H, D, dtype=torch.bfloat16, device=dev) for _ in range(2))

        def fn(_keep=(cu_dev, k, v, table, lens_dev)):
            nat.check(lib.pace_kv_gather_packed(ctypes.byref(cache._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias,
                                                cu_dev.data_ptr(), B, 1, k.data_ptr(), v.data_ptr(), int(cu[-1]), nat.current_stream_ptr()))
        return fn
    k, v = (torch.empty(B, H, L, D, dtype=torch.bfloat16, device=dev) for _ in range(2))
    if form == "dense":  # rows past each length left alone: launched over the blocks that exist, like the packed form
        cu = np.zeros(B + 1, dtype=np.int64)
        np.cumsum(cache.lens, out=cu[1:])
        cu_dev = torch.from_numpy(cu.astype(np.int32)).to(dev)

        def fn(_keep=(cu_dev, k, v, table, lens_dev)):
            nat.check(lib.pace_kv_gather_live(ctypes.byref(cache._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias,
                                              cu_dev.data_ptr(), B, 1, k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), L, int(cu[-1]),
                                              nat.current_stream_ptr()))
        return fn

    def fn(_keep=(k, v, table, lens_dev)):
        nat.check(lib.pace_kv_gather(ctypes.byref(cache._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias, B, 1,
                                     k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1), L, 1, nat.current_stream_ptr()))
    return fn


def wl_gather(torch, dev, args):
    """Block-table gather of the whole headline cache (batch 64 x 4096 tokens, permuted blocks) back into
    token rows: 2 x 1.07 GB of algorithmic traffic per call."""
    B, ctx, hq, hkv, D = 64, 4096, 32, 8, 128
    cache = build_cache(torch, dev, [ctx] * B, hq, hkv, D, seed=1, headroom=16)
    nbytes = 2 * B * ctx * kv_token_bytes(hkv, D)
    ms = {form: time_call(torch, gather_call(torch, cache, form), reps=args.steps, warmup=args.warmup) for form in ("dense", "packed")}
    return result_line(args, "block-table gather: batch 64 x 4096 tokens, 8 KV heads, head_dim 128, permuted blocks -> dense [B,H,L,D]",
                       nbytes, B * ctx, ms["dense"] * 1e-3, roofline("kv_gather_kernel<128,false> (dense)", nbytes, ms["dense"]),
                       extra={"packed": roofline("kv_gather_kernel<128,true> (packed)", nbytes, ms["packed"])})


def wl_append(torch, dev, args):
    """KV append on its own (not fused into the attention launch): T new tokens per sequence on top of the
    headline cache, T = 1 (decode), 8 (verify), 512 (prefill chunk).  Bytes = new K/V read + written."""
    from pace_mi355 import _native as nat

    B, ctx, hq, hkv, D = 64, 4096, 32, 8, 128
    cache = build_cache(torch, dev, [ctx] * B, hq, hkv, D, seed=1, headroom=512 + 16)
    lib = nat.load()
    g = torch.Generator(device=dev).manual_seed(3)
    res = {}
    for T in (1, 8, 512):
        k, v = _randn_bf16(torch, (B, hkv, T, D), g, dev), _randn_bf16(torch, (B, hkv, T, D), g, dev)
        lens_after = cache.lens + T
        cache.state.ensure_capacity(lens_after)
        table = cache.state.device_table()
        lens_dev = torch.from_numpy(lens_after.astype("int32")).to(dev)

        def fn():
            nat.check(lib.pace_kv_append_paged(ctypes.byref(cache._desc), k.data_ptr(), v.data_ptr(), k.stride(0), k.stride(1),
                                               k.stride(2), B, T, table.data_ptr(), table.stride(0), lens_dev.data_ptr(), -T,
                                               nat.current_stream_ptr()))
        ms = time_call(torch, fn, reps=args.steps, warmup=args.warmup)
        kernel = "kv_append_kernel<128,true>" if T < 8 else "kv_append_block_kernel<128,false>"
        res[T] = roofline(f"{kernel} ({T} tokens per sequence)", append_bytes(B, T, hkv, D), ms)
    return result_line(args, "KV append alone: batch 64, 8 KV heads, head_dim 128, 512 / 8 / 1 new tokens per sequence through the block "
                       "table (headline line: 512)", append_bytes(B, 512, hkv, D), B * 512, res[512]["avg_launch_ms"] * 1e-3, res[512],
                       extra={"append_8_tokens": res[8], "append_1_token": res[1]})


def wl_verify(torch, dev, args):
    import numpy as np

    B, hq, hkv, D, S = 32, 32, 8, 128, 8
    lens = np.random.default_rng(4).integers(1024, 8193, B).tolist()
    cache = build_cache(torch, dev, lens, hq, hkv, D, seed=4)
    cache.partition_tokens = args.partition
    g = torch.Generator(device=dev).manual_seed(5)
    kd, vd = _randn_bf16(torch, (B, hkv, S, D), g, dev), _randn_bf16(torch, (B, hkv, S, D), g, dev)
    q = _randn_bf16(torch, (B, hq, S, D), g, dev)
    step = FixedStep(torch, cache, q, kd, vd, args.partition, fused=not args.no_fuse)
    dt, attn_ms = run_timed(torch, step, args.steps, args.warmup)
    lens_v = [n + S for n in lens]
    dec = decode_bytes(lens_v, hq, hkv, D, q_len=S)
    flops = 4.0 * sum(lens_v) * hq * S * D
    check = {} if args.no_check else self_check(torch, step, spread_rows(lens_v))
    return result_line(
        args, "PARD speculative verify: batch 32, contexts U[1024,8192] (seed 4), 8 draft tokens appended + causal "
        "8-query attention", dec + append_bytes(B, S, hkv, D), B * S, dt,
        roofline(step.kernel + " (verify) + merge", dec, attn_ms,
                 {"mfma_tflops": round(flops / (attn_ms * 1e-3) / 1e12, 2), "work_items": step.n_items, "max_parts": step.max_parts}),
        extra=check)


def wl_prefill(torch, dev, args):
    """One chunk of a chunked prefill: 512 new tokens per sequence appended to 3584 cached ones, then
    causal attention of the chunk over the cache (the reference runs prefill as the same update_cache +
    attention pair with q_len = prompt length, pace/llm/models/llama.py:286-299)."""
    B, hq, hkv, D, past, S = 8, 32, 8, 128, 3584, 512
    B, past = args.batch or B, args.context or past  # --batch / --context: other batch sizes / cached lengths
    cache = build_cache(torch, dev, [past] * B, hq, hkv, D, seed=8, headroom=S + 64)
    cache.partition_tokens = args.partition
    g = torch.Generator(device=dev).manual_seed(9)
    kd, vd = _randn_bf16(torch, (B, hkv, S, D), g, dev), _randn_bf16(torch, (B, hkv, S, D), g, dev)
    q = _randn_bf16(torch, (B, hq, S, D), g, dev)
    mask = None
    if args.mask:  # the additive causal mask the reference's models pass along (llama.py:292-299), as a tensor
        ctx = past + S
        ar = torch.arange(ctx, device=dev)
        mask = torch.zeros(B, 1, S, ctx, device=dev, dtype=torch.bfloat16)
        mask.masked_fill_(ar[None, :] > ar[:S, None] + past, torch.finfo(torch.bfloat16).min)
    step = FixedStep(torch, cache, q, kd, vd, args.partition, fused=False, mask=mask)
    dt, attn_ms = run_timed(torch, step, args.steps, args.warmup)
    # causal: row s of the chunk reads past + s + 1 tokens
    flops = 4.0 * B * hq * D * sum(past + s + 1 for s in range(S))
    kv_once = decode_bytes([past + S] * B, hq, hkv, D, q_len=S)
    tflops = flops / (attn_ms * 1e-3) / 1e12
    return result_line(
        args, f"chunked prefill: batch {B}, 512-token chunk on top of {past} cached tokens, 32 Q / 8 KV heads, head_dim 128; "
        "block append + causal attention of the chunk", kv_once + append_bytes(B, S, hkv, D), B * S, dt,
        {"bound": "mfma", "kernel": step.kernel + (" (prefill chunk, explicit mask)" if args.mask else " (prefill chunk)"), "achieved": round(tflops, 1),
         "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
         "flops_per_launch": flops, "avg_launch_ms": round(attn_ms, 5),
         "hbm_gbs_if_kv_read_once": round(kv_once / (attn_ms * 1e-3) / 1e9, 1)},
        {"mask": bool(args.mask)})


def wl_dense_prefill(torch, dev, args):
    """The reference's own op at a prefill shape: torch.ops.pace.attention on dense [B, N, L, H] K/V with
    the additive causal [B, 1, S, L] mask that LlamaModel.forward builds (pace/llm/models/llama.py:284-310),
    as the JIT backend calls it (pace/ops/backends/jit.py:31-47).  The mask is additive and arbitrary, so
    every (row, key) pair is computed: 4*B*N*S*L*H flop."""
    import pace_mi355.ops  # noqa: F401  (defines the op)

    B, N, S, L, H = args.batch or 8, args.heads or 32, args.queries or 2048, args.context or 2048, args.head_dim or 128
    g = torch.Generator(device=dev).manual_seed(10)
    q, k, v = (_randn_bf16(torch, (B, N, n, H), g, dev) for n in (S, L, L))
    mask = torch.zeros(B, 1, S, L, device=dev, dtype=torch.bfloat16)
    ar = torch.arange(L, device=dev)
    mask.masked_fill_(ar[None, :] > ar[:S, None] + (L - S), torch.finfo(torch.bfloat16).min)

    def step(ev=None):
        if ev:
            ev[0].record()
        torch.ops.pace.attention(q, k, v, mask, False)
        if ev:
            ev[1].record()

    dt, attn_ms = run_timed(torch, step, args.steps, args.warmup)
    # flops the result needs: the pairs the causal mask leaves readable (row s reads L - S + s + 1 keys).  The
    # mask is an arbitrary additive tensor to the kernel, which only leaves out 32-key units that are at the
    # floor for all 32 rows of a wave; the rest of the masked half is computed and weighs zero.
    flops = 4.0 * B * N * H * sum(L - S + s + 1 for s in range(S))
    all_pairs = 4.0 * B * N * S * L * H
    once = 2 * (q.numel() * 2 + k.numel() + v.numel()) + B * S * L * 2  # q, out, K, V and the mask read once
    tflops = flops / (attn_ms * 1e-3) / 1e12
    return result_line(
        args, f"dense op at a prefill shape: batch {B}, {N} heads, {S} queries x {L} keys, head_dim {H}, additive causal mask "
        "[B,1,S,L]; step = one torch.ops.pace.attention call (output allocation included)", once, B * S, dt,
        {"bound": "mfma", "kernel": "dense_attn_coop_kernel<128,2,2>" if (H, S) == (128, 2048) else f"bf16 dense op, head_dim {H}, {S} query rows",
         "achieved": round(tflops, 1),
         "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
         "flops_per_launch": flops, "avg_launch_ms": round(attn_ms, 5),
         "tflops_if_all_pairs_counted": round(all_pairs / (attn_ms * 1e-3) / 1e12, 1)})


def wl_dense_f32(torch, dev, args):
    """The reference's own op on fp32 tensors (its tests' dtype, tests/ops/test_sdpa.py:83-127): the general
    kernel, fp32 arithmetic on the matrix cores.  Mask [B,1,1,L] as in the reference's test."""
    import pace_mi355.ops  # noqa: F401  (defines the op)

    B, N, S, L, H = 8, 32, 512, 512, 128
    g = torch.Generator(device=dev).manual_seed(11)
    q, k, v = (torch.randn(B, N, n, H, generator=g, device=dev) for n in (S, L, L))
    mask = torch.randn(B, 1, 1, L, generator=g, device=dev)

    def step(ev=None):
        if ev:
            ev[0].record()
        torch.ops.pace.attention(q, k, v, mask, False)
        if ev:
            ev[1].record()

    dt, attn_ms = run_timed(torch, step, args.steps, args.warmup)
    flops = 4.0 * B * N * S * L * H
    once = 4 * (2 * q.numel() + k.numel() + v.numel()) + 4 * mask.numel()
    tflops = flops / (attn_ms * 1e-3) / 1e12
    return result_line(
        args, "dense op on fp32 tensors: batch 8, 32 heads, 512 queries x 512 keys, head_dim 128, additive mask [B,1,1,L]; "
        "step = one torch.ops.pace.attention call (output allocation included)", once, B * S, dt,
        {"bound": "mfma", "kernel": "attn_f32_coop_kernel<float,128,false,true>", "achieved": round(tflops, 1),
         "peak": MFMA_F32_PEAK_TFLOPS, "unit": "TFLOP/s", "frac": round(tflops / MFMA_F32_PEAK_TFLOPS, 4), "traffic": None,
         "flops_per_launch": flops, "avg_launch_ms": round(attn_ms, 5)}, extra={"dtype": "f32"})


def wl_decode_f32pool(torch, dev, args):
    """The headline step for an fp32 model (the reference's caches keep the model's dtype,
    pace/llm/cache.py:255-266): a pool of fp32 rows, the 1-token append and the decode attention in one launch
    (--no-fuse: the append as a launch of its own)."""
    B, ctx, hq, hkv, D = args.batch or 64, args.context or 4096, 32, 8, 128
    cache = build_cache(torch, dev, [ctx] * B, hq, hkv, D, seed=1, permute=not args.no_permute, f32=True)
    g = torch.Generator(device=dev).manual_seed(2)
    k1, v1, q = (torch.randn(B, h, 1, D, generator=g, device=dev) for h in (hkv, hkv, hq))
    fused = not args.no_fuse
    fs = FixedStep(torch, cache, q, k1, v1, fused=fused)
    dt, attn_ms = run_timed(torch, fs, args.steps, args.warmup)
    nbytes = 2 * decode_bytes(fs.lens_after.tolist(), hq, hkv, D) - 4 * B - 4 * B * math.ceil((ctx + 1) / 16)  # fp32 rows, the same table
    app = 2 * append_bytes(B, 1, hkv, D)
    check = {}
    if not args.no_check:  # the step's output against the fp32 oracle (1e-5), the appended rows bit for bit
        from oracle.attention_ref import lengths_mask_4d, sdpa_fp32
        from oracle.cache_ref import repeat_kv

        torch.cuda.synchronize()
        gk, gv = fs.gathered()
        rows = [0, B // 2, B - 1]
        idx = torch.tensor(rows, device=dev)
        ref = sdpa_fp32(q[idx].cpu(), repeat_kv(gk[idx].cpu(), hq // hkv), repeat_kv(gv[idx].cpu(), hq // hkv),
                        lengths_mask_4d([ctx + 1] * len(rows), 1, ctx + 1, torch.float32))
        err = float((fs.out[idx].cpu() - ref).abs().max())
        slots = bool(torch.equal(gk[:, :, ctx], k1[:, :, 0]) and torch.equal(gv[:, :, ctx], v1[:, :, 0]))
        check = {"checked": bool(err <= 1e-5 and slots), "max_abs_err": err, "appended_slots_bit_exact": slots, "checked_sequences": rows,
                 "check": "last timed step vs the fp32 CPU oracle (cap 1e-5); slots of the new tokens bit-exact for every sequence"}
    return result_line(
        args, f"decode over a pool of fp32 rows: batch {B}, context {ctx} (+1 appended), 32 Q / 8 KV heads, head_dim 128, KV block 16, "
        f"seeded random physical block permutation, 1-token append + GQA decode ({'one launch' if fused else 'two launches'})",
        nbytes + app, B, dt, roofline(fs.kernel, nbytes + (app if fused else 0), attn_ms), extra=dict(check, dtype="f32"))


def wl_compact(torch, dev, args):
    import numpy as np

    B, hq, hkv, D, ctx = 8, 64, 8, 128, 32768
    g = torch.Generator(device=dev).manual_seed(7)
    q = _randn_bf16(torch, (B, hq, 1, D), g, dev)
    block_bytes = 16 * kv_token_bytes(hkv, D)
    times, walls, moved = [], [], 0
    for rep in range(3):  # compaction is destructive: rebuild, evict, then time one compaction
        cache = build_cache(torch, dev, [ctx] * B, hq, hkv, D, seed=6, headroom=0)
        rng = np.random.default_rng(6)
        for b in range(B):
            cache.evict_blocks(b, np.sort(rng.choice(ctx // 16, size=int(0.4 * ctx // 16), replace=False)).tolist())
        cache.state.upload_pairs(np.zeros((cache.state.allocator.num_blocks, 2), dtype=np.int32))  # a cache that lives on has its staging buffer already
        torch.cuda.synchronize()
        # PagedKVCache.compact(): one library call plans the moves (a pass over the table), uploads the (src, dst)
        # pairs and starts the copy; the table and the free list are rewritten while the GPU copies.  Here the same
        # steps on the wall clock (synchronize on both sides); the copy kernel alone is timed below.
        from pace_mi355 import _native as nat
        t_wall = time.perf_counter()
        moves = cache.state.compact_blocks([cache._desc])
        cache.state.apply_moves(moves)
        torch.cuda.synchronize()
        walls.append((time.perf_counter() - t_wall) * 1e3)
        moved = len(moves)
        # the copy kernel by itself: the same pairs once more (the moved blocks now hold the data; any source will do)
        pairs = cache.state._pairs_dev[:moved]
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        nat.check(nat.load().pace_kv_copy_blocks(ctypes.byref(cache._desc), ctypes.byref(cache._desc), pairs.data_ptr(),
                                                 moved, nat.current_stream_ptr()))
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    host_ms = min(walls)
    compact_ms = min(times)
    cache.partition_tokens = args.partition
    lens = cache.lens.tolist()
    dec = decode_bytes(lens, hq, hkv, D)
    attn_ms = time_call(torch, lambda: cache.attend(q), reps=args.steps, warmup=args.warmup)
    check = {}
    if not args.no_check:  # decode over the compacted cache against the oracle over the surviving tokens, gathered back
        gk, gv = cache.gather(n_rep=1)
        check = check_attention(torch, q, cache.attend(q), gk, gv, lens, [0, B - 1])
        used = np.concatenate([cache.state.table[b, : cache.state.n_blocks[b]] for b in range(B)])
        check["blocks_contiguous"] = bool(sorted(used.tolist()) == list(range(len(used))))
        check["checked"] = bool(check["checked"] and check["blocks_contiguous"])
        check["check"] = "decode after compaction vs the fp32 CPU oracle over the surviving tokens; live blocks occupy ids 0..n-1"
    return result_line(
        args, f"long-context compaction: 70B-shape KV (64 Q / 8 KV heads), batch 8, context 32768, 40% of blocks evicted "
        f"(seed 6), {moved} blocks moved, then decode over {lens[0]} tokens/seq", dec, B, attn_ms * 1e-3,
        roofline("paged_attn_kernel<128,1,...> (decode after compaction) + merge", dec, attn_ms),
        extra={"compaction": roofline("kv_copy_blocks_kernel", 2 * moved * block_bytes, compact_ms,
                                      {"blocks_moved": moved, "end_to_end_ms": round(host_ms, 3),
                                       "end_to_end_note": "plan + upload + copy + table rewrite, wall clock between two synchronizes"}),
               **check})


def wl_copy_calibration(torch, dev, args):
    """Copies N whole blocks (N x 64 KiB read, N x 64 KiB written): the known-size kernel the
    HBM byte counters are scaled by."""
    from pace_mi355 import _native as nat

    hq, hkv, D, N = 32, 8, 128, 8192
    cache = build_cache(torch, dev, [16 * 2 * N // 64] * 64, hq, hkv, D, seed=9, headroom=0)
    pairs = torch.stack([torch.arange(0, N, dtype=torch.int32), torch.arange(N, 2 * N, dtype=torch.int32)], 1).to(dev)
    lib = nat.load()

    def copy():
        nat.check(lib.pace_kv_copy_blocks(ctypes.byref(cache._desc), ctypes.byref(cache._desc), pairs.data_ptr(), N,
                                          nat.current_stream_ptr()))

    ms = time_call(torch, copy, reps=args.steps, warmup=args.warmup)
    nbytes = 2 * N * 16 * kv_token_bytes(hkv, D)
    return result_line(args, f"block copy calibration: {N} blocks of 64 KiB, disjoint src/dst", nbytes, 0, ms * 1e-3,
                       roofline("kv_copy_blocks_kernel", nbytes, ms, {"bytes_read": nbytes // 2, "bytes_written": nbytes // 2}))


def cpu_baseline(torch, batch, ctx, hq, hkv, D, warmup=2, timed=5):
    """The reference's CPU path, restated by the oracle, at the full batch of the workload: GQA-expanded K/V
    in the reference's cache + torch CPU SDPA in bf16 (pace/llm/models/llama.py:151-165).  Two legs: the BMC
    cache its benchmark configuration selects (benchmarks/llm/performance/benchmark_config.json) and the
    DYNAMIC cache its generator defaults to (pace/llm/llm.py:59), whose torch.cat re-copies the whole cache on
    every step (pace/llm/cache.py:391-395).  2 warm-up + 5 timed steps, as the reference's benchmark runs
    (benchmark_config.json:29-30)."""
    from oracle.attention_ref import lengths_mask_4d, sdpa_native
    from oracle.cache_ref import BMCKVCacheRef, DynamicKVCacheRef, repeat_kv

    cores = torch.get_num_threads()
    B, n_rep = batch, hq // hkv
    g = torch.Generator().manual_seed(0)
    k = torch.randn(B, hkv, ctx, D, generator=g).to(torch.bfloat16)
    v = torch.randn(B, hkv, ctx, D, generator=g).to(torch.bfloat16)
    k1 = torch.randn(B, hkv, 1, D, generator=g).to(torch.bfloat16)
    v1 = torch.randn(B, hkv, 1, D, generator=g).to(torch.bfloat16)
    q = torch.randn(B, hq, 1, D, generator=g).to(torch.bfloat16)
    nbytes = decode_bytes([ctx + 1] * B, hq, hkv, D) + append_bytes(B, 1, hkv, D)
    legs = {}
    for name, cls in (("bmc", BMCKVCacheRef), ("dynamic", DynamicKVCacheRef)):
        cache = cls(ctx + 128)
        cache.update_cache(repeat_kv(k, n_rep).contiguous(), repeat_kv(v, n_rep).contiguous(), 2)

        def step():
            ke, ve = repeat_kv(k1, n_rep), repeat_kv(v1, n_rep)
            K, V = cache.update_cache(ke, ve, 2)
            n = cache.seq_len
            mask = cache.update_mask(lengths_mask_4d([n] * B, 1, n, torch.bfloat16), n)
            out = sdpa_native(q, K, V, mask)
            cache.remove_cache(1)  # every step runs at the same cache state, like the GPU line
            return out

        for _ in range(warmup):
            step()
        t0 = time.perf_counter()
        for _ in range(timed):
            step()
        dt = (time.perf_counter() - t0) / timed
        legs[name] = {"value": round(nbytes / dt / 1e9, 3), "tokens_per_s": round(B / dt, 2), "ms_per_step": round(dt * 1e3, 3)}
        del cache
    return {
        "value": legs["bmc"]["value"],
        "unit": "GB/s",
        "tokens_per_s": legs["bmc"]["tokens_per_s"],
        "ms_per_step": legs["bmc"]["ms_per_step"],
        "cores": cores,
        "kind": "port",
        "sample": f"the whole workload: batch {B}, context {ctx}, BMC cache with GQA-expanded K/V + torch CPU SDPA bf16; "
                  f"{warmup} warm-up + {timed} timed steps; GB/s uses the same GQA-minimal algorithmic bytes as the GPU line",
        "dynamic_cache": dict(legs["dynamic"], note="the same step with the reference's default DYNAMIC cache (torch.cat of the "
                                                    "whole cache per step)"),
    }


def other_configs(torch, dev, args):
    """Short legs over the other benchmark configurations (the ragged serving mix, the speculative verify step, the
    long-context compaction), at most 20 timed steps each, so that one default run carries every configuration's
    roofline figure.  `value` of the line stays the headline workload's."""
    import copy
    import gc

    out = {}
    for name in ("ragged", "verify", "compact"):
        a = copy.copy(args)
        a.steps, a.warmup, a.workload = min(args.steps, 20), min(args.warmup, 5), name
        gc.collect()
        torch.cuda.empty_cache()
        res = WORKLOADS[name](torch, dev, a)
        keep = {k: res[k] for k in ("value", "unit", "pct_of_hbm_peak", "tokens_per_s", "steps", "warmup", "ms_per_step", "roofline",
                                    "checked", "max_abs_err", "max_rel_err", "appended_slots_bit_exact", "checked_sequences",
                                    "gather", "compaction", "blocks_contiguous") if k in res}
        keep["workload"] = res["config"]["workload"]
        keep["bytes_per_step"] = res["config"]["bytes_per_step"]
        out[name] = keep
    gc.collect()
    torch.cuda.empty_cache()
    return out


WORKLOADS = {"gather": wl_gather, "append": wl_append, "decode-8b": wl_decode_8b, "decode-gptj": wl_decode_gptj, "ragged": wl_ragged, "verify": wl_verify, "prefill": wl_prefill, "dense-f32": wl_dense_f32, "decode-f32pool": wl_decode_f32pool,
             "dense-prefill": wl_dense_prefill, "compact": wl_compact, "copy-calibration": wl_copy_calibration}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--workload", choices=sorted(WORKLOADS), default="decode-8b")
    ap.add_argument("--path", choices=("api", "direct", "graph"), default="direct",
                    help="decode workloads. direct: C-ABI calls with fixed metadata; api: PagedKVCache.update_cache + "
                         "MultiHeadAttention; graph: the api calls captured once into a HIP graph and replayed per step")
    ap.add_argument("--batch", type=int, default=0, help="decode and prefill workloads: override the batch size (latency studies)")
    ap.add_argument("--context", type=int, default=0, help="decode and prefill workloads: override the context length (prefill: the cached tokens)")
    ap.add_argument("--heads", type=int, default=0, help="dense-prefill: number of heads (default 32)")
    ap.add_argument("--head-dim", type=int, default=0, dest="head_dim", help="dense-prefill: head size (default 128)")
    ap.add_argument("--queries", type=int, default=0, help="dense-prefill: query rows per head (default 2048; --context gives the keys)")
    ap.add_argument("--layers", type=int, default=4,
                    help="decode workloads: distinct layer pools (own block permutation each) the timed steps rotate over; "
                         "4 x 1.07 GB is 16 times the last-level cache, 1 re-reads one pool every step")
    ap.add_argument("--partition", type=int, default=0, help="context split size in tokens (0 = library default)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true", dest="no_check",
                    help="skip the comparison of the last step's results with the CPU oracle after the timed region")
    ap.add_argument("--no-others", action="store_true", dest="no_others",
                    help="default workload only: skip the short legs over the other configurations (ragged, verify, compact)")
    ap.add_argument("--mask", action="store_true",
                    help="decode-8b, api path: pass repeat_kv-expanded K/V and the step's additive mask, as the reference's "
                         "models call the cache and the attention operator; prefill: pass the causal mask as a tensor")
    ap.add_argument("--rope", action="store_true",
                    help="decode-8b, direct path: q and k arrive un-rotated and the rotary embedding rides in the launch "
                         "(with --no-fuse: in the append launch)")
    ap.add_argument("--no-fuse", action="store_true",
                    help="launch the append as its own kernel instead of fusing it into the attention launch")
    ap.add_argument("--no-permute", action="store_true", help="keep physical blocks in logical order (diagnostic)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the hot path shards by sequence or by KV "
              "head with no exchange). Run with --gpus 1.", file=sys.stderr)
        return 2
    import torch

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    line = WORKLOADS[args.workload](torch, dev, args)
    plain_default = (args.workload == "decode-8b" and args.path == "direct" and not (args.batch or args.context or args.rope or args.mask
                                                                                    or args.no_fuse or args.no_permute or args.partition))
    if plain_default and not args.no_others:
        line["others"] = other_configs(torch, dev, args)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
