"""The entry points only enqueue kernels on the stream they are given -- no allocation, no
memset, no host synchronisation -- so a decode step can be captured into a HIP graph and
replayed.  Replays are checked against the eager result with eager work in between."""
import ctypes
import math

import pytest
import torch

from helpers import assert_bits_equal, seeded_kv, seeded_q

pytestmark = pytest.mark.gpu


def _frozen_step(cache, q, k_new, v_new, out, ws, rope=None):
    """C-ABI call with every argument fixed: one new token per sequence on top of the cache as it is."""
    from pace_mi355 import _native as nat

    lib = nat.load()
    B, hq, S, D = q.shape
    T = k_new.shape[2]
    st = cache.state
    lens_after = cache.lens + T
    st.ensure_capacity(lens_after)
    table = st.device_table()
    lens_dev = torch.from_numpy(lens_after.astype("int32")).to(q.device)
    a = nat.PagedAttnArgs()
    a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
    a.block_table, a.table_stride, a.seq_lens = table.data_ptr(), table.stride(0), lens_dev.data_ptr()
    a.causal, a.batch, a.num_q_heads, a.q_len = 1, B, hq, S
    a.max_seq_len, a.partition_tokens, a.scale = int(lens_after.max()), 256, 1.0 / math.sqrt(D)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.k_new, a.v_new, a.n_new = k_new.data_ptr(), v_new.data_ptr(), T
    a.new_stride_b, a.new_stride_h, a.new_stride_t = k_new.stride(0), k_new.stride(1), k_new.stride(2)
    if rope is not None:
        a.rope = ctypes.pointer(rope)
    keep = (table, lens_dev, a, rope)

    def launch():
        fn = lib.pace_paged_attn_decode if S == 1 else lib.pace_paged_attn_verify
        nat.check(fn(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))

    return launch, keep


@pytest.mark.parametrize("S", [1, 4])
def test_decode_step_replays_from_a_hip_graph(device, S):
    from pace_mi355.llm import PagedKVCache

    B, hkv, n_rep, D = 4, 2, 4, 128
    lens = [700, 33, 1500, 256]  # several partitions: the merge kernel is part of the graph
    cache = PagedKVCache(2048, num_kv_heads=hkv, n_rep=n_rep)
    k, v = seeded_kv(1, B, hkv, max(lens), D)
    cache.append_ragged(k.to(device), v.to(device), lens)
    q = seeded_q(2, B, hkv * n_rep, S, D).to(device)
    k1, v1 = (t.to(device) for t in seeded_kv(3, B, hkv, S, D))
    out = torch.zeros(B, hkv * n_rep, S, D, dtype=torch.bfloat16, device=device)
    ws = torch.empty(8 << 20, dtype=torch.uint8, device=device)
    launch, keep = _frozen_step(cache, q, k1, v1, out, ws)
    launch()
    torch.cuda.synchronize()
    eager = out.clone()

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        launch()  # warm-up on the capture stream
        side.synchronize()
        with torch.cuda.graph(graph, stream=side):
            launch()
    for i in range(4):
        out.zero_()
        q_scratch = torch.randn(1 << 16, device=device).sum()  # unrelated eager work between replays
        graph.replay()
        torch.cuda.synchronize()
        assert_bits_equal(out, eager, f"replay {i}")
        assert torch.isfinite(q_scratch)
    # new inputs in the same buffers are picked up by the next replay
    q.copy_(seeded_q(9, B, hkv * n_rep, S, D))
    launch()
    torch.cuda.synchronize()
    eager2 = out.clone()
    out.zero_()
    graph.replay()
    torch.cuda.synchronize()
    assert_bits_equal(out, eager2, "replay with new query")
    assert not torch.equal(eager2, eager)


def test_captured_decode_loop_advances_lengths_on_the_device(device):
    """A whole decode loop from one captured step: the graph holds the fused append + attention
    launch and a one-element increment of the device-side length addend, so every replay appends
    at the next position and attends over one more token.  No host-side argument changes."""
    from oracle.paged_ref import RaggedCacheModel
    from pace_mi355 import _native as nat
    from pace_mi355.llm import PagedKVCache

    B, hkv, n_rep, D, steps = 3, 2, 4, 128, 40
    lens0 = [100, 17, 333]
    cache = PagedKVCache(512, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, D)
    k, v = seeded_kv(1, B, hkv, max(lens0), D)
    cache.append_ragged(k.to(device), v.to(device), lens0)
    model.append(k, v, lens0)
    st = cache.state
    st.ensure_capacity(cache.lens + steps)           # blocks for every future position, before capture
    table = st.device_table()
    lens_dev = torch.tensor(lens0, dtype=torch.int32, device=device)
    step_no = torch.zeros(1, dtype=torch.int32, device=device)
    q = torch.zeros(B, hkv * n_rep, 1, D, dtype=torch.bfloat16, device=device)
    k1, v1 = torch.zeros(B, hkv, 1, D, dtype=torch.bfloat16, device=device), torch.zeros(B, hkv, 1, D, dtype=torch.bfloat16, device=device)
    out = torch.zeros_like(q)
    ws = torch.empty(4 << 20, dtype=torch.uint8, device=device)
    lib = nat.load()
    a = nat.PagedAttnArgs()
    a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
    a.block_table, a.table_stride, a.seq_lens = table.data_ptr(), table.stride(0), lens_dev.data_ptr()
    a.seq_len_bias, a.seq_len_bias_ptr = 1, step_no.data_ptr()   # length = lens0 + 1 + steps done so far
    a.causal, a.batch, a.num_q_heads, a.q_len = 1, B, hkv * n_rep, 1
    a.max_seq_len, a.partition_tokens, a.scale = max(lens0) + steps, 128, 1.0 / math.sqrt(D)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    a.k_new, a.v_new, a.n_new = k1.data_ptr(), v1.data_ptr(), 1
    a.new_stride_b, a.new_stride_h, a.new_stride_t = k1.stride(0), k1.stride(1), k1.stride(2)

    def launch():
        nat.check(lib.pace_paged_attn_decode(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))
        step_no.add_(1)

    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            launch()
    for i in range(steps):
        kn, vn = seeded_kv(100 + i, B, hkv, 1, D)
        qn = seeded_q(200 + i, B, hkv * n_rep, 1, D)
        k1.copy_(kn), v1.copy_(vn), q.copy_(qn)
        graph.replay()
        model.append(kn, vn)
        if i % 7 == 0 or i == steps - 1:
            torch.cuda.synchronize()
            from helpers import assert_attention_close
            assert_attention_close(out, model.attention(qn, n_rep), f"replay {i}")
    torch.cuda.synchronize()
    assert int(step_no.item()) == steps
    cache.lens = cache.lens + steps
    cache.seq_len = int(cache.lens.max())
    gk, gv = cache.gather(n_rep=1)
    K, V = model.dense(1)
    assert_bits_equal(gk, K, "pool K after the captured loop")
    assert_bits_equal(gv, V, "pool V after the captured loop")


def test_manager_decode_step_captured_once_and_replayed_per_token(device):
    """KVCacheManager.capture_decode: the whole decode step of a two-layer model -- per layer update_cache +
    MultiHeadAttention on static tensors -- captured once, replayed per token with nothing but the inputs
    changing; lengths advance on the device.  Attention against the oracle every step, cache contents bit-exact
    at the end; any other cache operation ends the graph and step-by-step operation carries on."""
    from oracle.paged_ref import RaggedCacheModel
    from pace_mi355.llm import KVCacheManager, KVCacheType
    from pace_mi355.ops import MultiHeadAttention

    class Cfg:
        num_hidden_layers = 2
        num_attention_heads = 8
        num_key_value_heads = 2

    B, hkv, n_rep, D, steps = 3, 2, 4, 128, 70   # 70 steps cross the 64-token buckets an eager plan is kept for
    lens0 = [300, 17, 1200]
    mgr = KVCacheManager(Cfg(), 2048, KVCacheType.PAGED)
    models = [RaggedCacheModel(B, hkv, D) for _ in range(2)]
    for layer in range(2):
        k, v = seeded_kv(10 + layer, B, hkv, max(lens0), D)
        mgr[layer].append_ragged(k.to(device), v.to(device), lens0)
        models[layer].append(k, v, lens0)
    mha = MultiHeadAttention(dtype=torch.bfloat16)
    qs = [torch.zeros(B, hkv * n_rep, 1, D, dtype=torch.bfloat16, device=device) for _ in range(2)]
    ks = [torch.zeros(B, hkv, 1, D, dtype=torch.bfloat16, device=device) for _ in range(2)]
    vs = [torch.zeros(B, hkv, 1, D, dtype=torch.bfloat16, device=device) for _ in range(2)]

    def step():
        outs = []
        for layer in range(2):
            pk, pv = mgr[layer].update_cache(ks[layer], vs[layer], 2)
            outs.append(mha(qs[layer], pk, pv))
        return outs

    graph = mgr.capture_decode(step, max_steps=steps)
    assert len(mgr) == max(lens0), "capturing leaves the cache as it was"
    for i in range(steps):
        new = []
        for layer in range(2):
            kn, vn = seeded_kv(1000 + 2 * i + layer, B, hkv, 1, D)
            qn = seeded_q(2000 + 2 * i + layer, B, hkv * n_rep, 1, D)
            ks[layer].copy_(kn), vs[layer].copy_(vn), qs[layer].copy_(qn)
            models[layer].append(kn, vn)
            new.append(qn)
        outs = graph.replay()
        assert len(mgr) == max(lens0) + i + 1
        if i % 9 == 0 or i == steps - 1:
            from helpers import assert_attention_close
            for layer in range(2):
                assert_attention_close(outs[layer], models[layer].attention(new[layer], n_rep), f"replay {i} layer {layer}")
    with pytest.raises(RuntimeError, match="reserved blocks for"):
        graph.replay()
    for layer in range(2):
        K, V = models[layer].dense(1)
        gk, gv = mgr[layer].gather(n_rep=1)
        assert_bits_equal(gk, K, f"pool K of layer {layer}")
        assert_bits_equal(gv, V, f"pool V of layer {layer}")
    # a second graph, ended early by a rollback; the eager path carries on from there
    graph = mgr.capture_decode(step, max_steps=8)
    for layer in range(2):
        kn, vn = seeded_kv(5000 + layer, B, hkv, 1, D)
        ks[layer].copy_(kn), vs[layer].copy_(vn)
        models[layer].append(kn, vn)
    graph.replay()
    mgr.remove_cache(1)
    for m in models:
        m.truncate([1] * B)
    with pytest.raises(RuntimeError, match="spent"):
        graph.replay()
    outs = step()
    for layer in range(2):
        models[layer].append(ks[layer].cpu(), vs[layer].cpu())
        from helpers import assert_attention_close
        assert_attention_close(outs[layer], models[layer].attention(qs[layer].cpu(), n_rep), f"eager step after the graph, layer {layer}")


def test_a_step_that_is_not_the_captured_kind_is_refused(device):
    """A step that does more on a cache than one update_cache + attention per layer would make the capture record
    uploads of host data (stale on replay): the eager run shows it and the capture is refused; a step that only
    departs from its eager run while it is being captured raises inside the capture.  The cache works on
    step by step afterwards."""
    from oracle.paged_ref import RaggedCacheModel
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.llm.graph import DecodeGraph

    B, hkv, n_rep, D = 2, 2, 4, 128
    cache = PagedKVCache(512, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, D)
    k, v = seeded_kv(1, B, hkv, 100, D)
    cache.append_ragged(k.to(device), v.to(device), [100, 40])
    model.append(k, v, [100, 40])
    k1, v1 = (t.to(device) for t in seeded_kv(2, B, hkv, 1, D))
    q = seeded_q(3, B, hkv * n_rep, 1, D).to(device)

    def two_updates():  # the second update of the layer flushes the first: not a captured step
        cache.update_cache(k1, v1, 2)
        cache.update_cache(k1, v1, 2)
        return cache.attend(q)

    with pytest.raises(RuntimeError, match="cannot be captured"):
        DecodeGraph([cache], two_updates, 4)
    assert cache._graph is None and cache.lens.tolist() == [100, 40], "a refused capture leaves the cache as it was"

    calls = [0]

    def changes_its_mind():  # eager run: a proper step; under capture: a gather in the middle
        calls[0] += 1
        cache.update_cache(k1, v1, 2)
        if calls[0] == 2:
            cache.gather()
        return cache.attend(q)

    with pytest.raises(RuntimeError, match="differs from its eager run"):
        DecodeGraph([cache], changes_its_mind, 4)
    torch.cuda.synchronize()
    assert cache._graph is None and cache.lens.tolist() == [100, 40] and cache._pending is None
    # step by step from here, as if nothing had happened
    cache.update_cache(k1, v1, 2)
    model.append(k1.cpu(), v1.cpu())
    from helpers import assert_attention_close
    assert_attention_close(cache.attend(q), model.attention(q.cpu(), n_rep), "eager step after the refused captures")
    K, V = model.dense(1)
    gk, gv = cache.gather(n_rep=1)
    assert_bits_equal(gk, K, "pool K")
    assert_bits_equal(gv, V, "pool V")
