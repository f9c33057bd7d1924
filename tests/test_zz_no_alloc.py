"""pace_paged_attn_verify_static: the entry point that allocates nothing.  Its partials live in an
array inside the library's device image instead of a caller workspace; everything else is the code
of pace_paged_attn_verify, so the two must agree bit for bit.  Two calls in a row share the array, the
second with a smaller input; a launch whose partials exceed the array is refused."""
import ctypes
import gc
import math

import pytest
import torch

from helpers import assert_attention_close, assert_bits_equal, seeded_kv, seeded_q

pytestmark = pytest.mark.gpu


def _args(nat, cache, q, out, partition, ws=None):
    B, hq, S, D = q.shape
    st = cache.state
    table = st.device_table()
    lens_dev = torch.from_numpy(cache.lens.astype("int32")).to(q.device)
    a = nat.PagedAttnArgs()
    a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
    a.block_table, a.table_stride, a.seq_lens = table.data_ptr(), table.stride(0), lens_dev.data_ptr()
    a.causal, a.batch, a.num_q_heads, a.q_len = 1, B, hq, S
    a.max_seq_len, a.partition_tokens, a.scale = int(cache.lens.max()), partition, 1.0 / math.sqrt(D)
    if ws is not None:
        a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    return a, (table, lens_dev)


def _both(device, seed, B, hkv, n_rep, D, S, lens, partition):
    """(output through the caller's workspace, output through the static array, oracle)."""
    from oracle.paged_ref import RaggedCacheModel
    from pace_mi355 import _native as nat
    from pace_mi355.llm import PagedKVCache

    lib = nat.load()
    cache = PagedKVCache(max(lens) + 16, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, D)
    k, v = seeded_kv(seed, B, hkv, max(lens), D)
    cache.append_ragged(k.to(device), v.to(device), lens)
    model.append(k, v, lens)
    q_host = seeded_q(seed + 1, B, hkv * n_rep, S, D)
    q = q_host.to(device)
    need = int(lib.pace_paged_attn_workspace_bytes(B, hkv * n_rep, S, D, max(lens), partition, hkv))
    assert 0 < need <= nat.STATIC_SCRATCH_BYTES, "the case must use partials, and they must fit the array"
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    out_ws = torch.zeros(B, hkv * n_rep, S, D, dtype=torch.bfloat16, device=device)
    out_static = torch.zeros_like(out_ws)
    a, keep = _args(nat, cache, q, out_ws, partition, ws)
    nat.check(lib.pace_paged_attn_verify(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))
    b, keep2 = _args(nat, cache, q, out_static, partition)  # no workspace at all
    # Device memory as the driver counts it (hipMemGetInfo), around a call that follows a warm-up call (code object
    # and symbol look-up are behind it): a hipMalloc inside the entry point would show here; torch's own counters
    # would not, the library never goes through torch's allocator.
    nat.check(lib.pace_paged_attn_verify_static(ctypes.byref(cache._desc), ctypes.byref(b), nat.current_stream_ptr()))
    torch.cuda.synchronize()
    out_static.zero_()
    gc.collect()  # tensors of earlier tests that are still waiting for the collector would be freed in between
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    nat.check(lib.pace_paged_attn_verify_static(ctypes.byref(cache._desc), ctypes.byref(b), nat.current_stream_ptr()))
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, f"device memory in use changed by {free_before - free_after} bytes across the call"
    return out_ws, out_static, model.attention(q_host, n_rep)


def test_static_scratch_entry_point_matches_the_workspace_one_on_two_calls_in_a_row(device):
    # first call: 4 sequences of up to 3000 tokens, 8 query tokens, partitions of 256 tokens -> 12 partials per row
    first = _both(device, 11, B=4, hkv=2, n_rep=4, D=128, S=8, lens=[3000, 517, 1999, 64], partition=256)
    assert_bits_equal(first[1], first[0], "first call")
    assert_attention_close(first[1], first[2], "first call vs oracle")
    # second call, smaller in every extent: the array still holds the first call's partials
    second = _both(device, 23, B=2, hkv=2, n_rep=4, D=128, S=1, lens=[700, 300], partition=128)
    assert_bits_equal(second[1], second[0], "second call")
    assert_attention_close(second[1], second[2], "second call vs oracle")


def test_static_scratch_entry_point_refuses_what_does_not_fit(device):
    from pace_mi355 import _native as nat
    from pace_mi355.llm import PagedKVCache

    lib = nat.load()
    B, hkv, n_rep, D, S = 16, 8, 4, 128, 32
    cache = PagedKVCache(4096 + 16, num_kv_heads=hkv, n_rep=n_rep)
    k, v = seeded_kv(5, B, hkv, 4096, D)
    cache.append_ragged(k.to(device), v.to(device), [4096] * B)
    q = seeded_q(6, B, hkv * n_rep, S, D).to(device)
    out = torch.full((B, hkv * n_rep, S, D), 7.0, dtype=torch.bfloat16, device=device)
    assert int(lib.pace_paged_attn_workspace_bytes(B, hkv * n_rep, S, D, 4096, 128, hkv)) > nat.STATIC_SCRATCH_BYTES
    a, keep = _args(nat, cache, q, out, 128)
    rc = lib.pace_paged_attn_verify_static(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr())
    assert rc == -1
    msg = lib.pace_kv_last_error().decode()
    assert "static buffer holds" in msg and "pace_paged_attn_verify_static" in msg
    torch.cuda.synchronize()
    assert bool((out == 7.0).all()), "nothing may have been launched"


def test_static_scratch_entry_point_with_a_mask_on_more_than_64_rows(device):
    """A masked launch of more than 64 query rows per KV head keeps its per-row mask summary behind the partials in
    the same array: same bits as the workspace entry point given a workspace of the array's size."""
    from oracle.attention_ref import sdpa_fp32
    from oracle.cache_ref import repeat_kv
    from pace_mi355 import _native as nat
    from pace_mi355.llm import PagedKVCache

    lib = nat.load()
    B, hkv, n_rep, D, S, L = 2, 2, 4, 128, 24, 600   # 96 query rows per KV head
    cache = PagedKVCache(L + 16, num_kv_heads=hkv, n_rep=n_rep)
    k, v = seeded_kv(31, B, hkv, L, D)
    cache.append_ragged(k.to(device), v.to(device), [L] * B)
    q_host = seeded_q(32, B, hkv * n_rep, S, D)
    q = q_host.to(device)
    # additive causal mask with some finite values mixed in (a line that is not "plain")
    ar = torch.arange(L)
    mask = torch.zeros(B, 1, S, L)
    mask.masked_fill_(ar[None, :] > ar[:S, None] + (L - S), torch.finfo(torch.bfloat16).min)
    mask[:, :, :, 5] = -1.5
    mask_dev = mask.to(torch.bfloat16).to(device)
    outs = []
    for static in (False, True):
        out = torch.zeros(B, hkv * n_rep, S, D, dtype=torch.bfloat16, device=device)
        ws = None if static else torch.empty(nat.STATIC_SCRATCH_BYTES, dtype=torch.uint8, device=device)
        a, keep = _args(nat, cache, q, out, 128, ws)
        a.mask, a.mask_dtype, a.mask_len, a.causal = mask_dev.data_ptr(), nat.DTYPE_BF16, L, 0
        a.mask_stride_b, a.mask_stride_s = mask_dev.stride(0), mask_dev.stride(2)
        fn = lib.pace_paged_attn_verify_static if static else lib.pace_paged_attn_verify
        nat.check(fn(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))
        torch.cuda.synchronize()
        outs.append(out)
    assert_bits_equal(outs[1], outs[0], "masked, 96 rows per KV head")
    ref = sdpa_fp32(q_host, repeat_kv(k, n_rep), repeat_kv(v, n_rep), mask.to(torch.bfloat16).float())
    assert_attention_close(outs[1], ref, "masked static launch vs oracle")


def test_static_scratch_entry_point_over_a_pool_of_fp32_rows(device):
    """A small batch over an fp32 pool is cut over several workgroups through the array (its own partial layout)."""
    from oracle.attention_ref import lengths_mask_4d, sdpa_fp32
    from oracle.cache_ref import repeat_kv
    from pace_mi355 import _native as nat
    from pace_mi355.llm import PagedKVCache

    lib = nat.load()
    B, hkv, n_rep, D, S, L = 2, 2, 4, 128, 1, 2048
    g = torch.Generator().manual_seed(41)
    k, v = torch.randn(B, hkv, L, D, generator=g), torch.randn(B, hkv, L, D, generator=g)
    q_host = torch.randn(B, hkv * n_rep, S, D, generator=g)
    cache = PagedKVCache(L + 16, num_kv_heads=hkv, n_rep=n_rep)
    cache.append_ragged(k.to(device), v.to(device), [L] * B)
    assert cache.f32
    q = q_host.to(device)
    outs = []
    for static in (False, True):
        out = torch.zeros(B, hkv * n_rep, S, D, dtype=torch.float32, device=device)
        ws = None if static else torch.empty(nat.STATIC_SCRATCH_BYTES, dtype=torch.uint8, device=device)
        a, keep = _args(nat, cache, q, out, 0, ws)
        fn = lib.pace_paged_attn_verify_static if static else lib.pace_paged_attn_verify
        nat.check(fn(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))
        torch.cuda.synchronize()
        outs.append(out)
    assert torch.equal(outs[1], outs[0]), "fp32 pool: the two entry points must give the same bits"
    ref = sdpa_fp32(q_host, repeat_kv(k, n_rep), repeat_kv(v, n_rep), lengths_mask_4d([L] * B, S, L, torch.float32))
    assert torch.allclose(outs[1].cpu(), ref, atol=1e-5, rtol=1e-5), (outs[1].cpu() - ref).abs().max()
    # the same launch without any workspace is one workgroup per (row group, KV head, sequence): the cut launch must
    # agree with it to rounding, which shows that the array was really used for partials
    out1 = torch.zeros_like(outs[0])
    a, keep = _args(nat, cache, q, out1, 0, None)
    nat.check(lib.pace_paged_attn_verify(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))
    torch.cuda.synchronize()
    assert torch.allclose(out1, outs[1], atol=1e-5, rtol=1e-5)


def test_static_scratch_entry_point_captured_into_a_graph(device):
    """The entry point under HIP graph capture (after an eager warm-up call, as the header asks): replayed twice with
    changed queries, each replay equals pace_paged_attn_verify on the same inputs bit for bit."""
    from pace_mi355 import _native as nat
    from pace_mi355.llm import PagedKVCache

    lib = nat.load()
    B, hkv, n_rep, D, S = 3, 2, 4, 128, 4
    lens = [1500, 700, 90]
    cache = PagedKVCache(max(lens) + 16, num_kv_heads=hkv, n_rep=n_rep)
    k, v = seeded_kv(51, B, hkv, max(lens), D)
    cache.append_ragged(k.to(device), v.to(device), lens)
    q = seeded_q(52, B, hkv * n_rep, S, D).to(device)  # static input buffer of the graph
    out = torch.zeros(B, hkv * n_rep, S, D, dtype=torch.bfloat16, device=device)
    need = int(lib.pace_paged_attn_workspace_bytes(B, hkv * n_rep, S, D, max(lens), 256, hkv))
    assert 0 < need <= nat.STATIC_SCRATCH_BYTES
    a, keep = _args(nat, cache, q, out, 256)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        nat.check(lib.pace_paged_attn_verify_static(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))  # warm-up
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            nat.check(lib.pace_paged_attn_verify_static(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    ws = torch.empty(need, dtype=torch.uint8, device=device)
    for rep in range(3):
        q.copy_(seeded_q(60 + rep, B, hkv * n_rep, S, D).to(device))
        out.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = torch.zeros_like(out)
        b, keep2 = _args(nat, cache, q, want, 256, ws)
        nat.check(lib.pace_paged_attn_verify(ctypes.byref(cache._desc), ctypes.byref(b), nat.current_stream_ptr()))
        torch.cuda.synchronize()
        assert_bits_equal(out, want, f"replay {rep}")
