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
    gc.collect()  # tensors of earlier tests that are still waiting for the collector would be freed in between
    before = torch.cuda.memory_allocated()
    nat.check(lib.pace_paged_attn_verify_static(ctypes.byref(cache._desc), ctypes.byref(b), nat.current_stream_ptr()))
    assert torch.cuda.memory_allocated() <= before, "the entry point took memory from torch's allocator"
    torch.cuda.synchronize()
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
