"""GPU parity: rotary embedding (dense, rotate-and-append, folded into the attention launch)
against the CPU restatement of the reference operator.  Rotated rows are bf16 tensor
arithmetic in the reference, so they must match bit for bit; attention within the
hot path's tolerance."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_attention_close, assert_bits_equal, seeded_kv, seeded_q
from oracle import rope_ref
from oracle.attention_ref import sdpa_fp32
from oracle.cache_ref import DynamicKVCacheRef, repeat_kv

pytestmark = pytest.mark.gpu


def _module(D, rows=512, scaling=None, theta=10000.0, **kw):
    from pace_mi355.ops import RotaryEmbedding

    return RotaryEmbedding(scaling, D, rows, theta, **kw)


def _oracle_rotate(x, module, position_ids, neox=True):
    cos, sin = rope_ref.lookup(module.cos_cache, module.sin_cache, position_ids, x.dtype)
    return rope_ref.rotate(x, cos, sin, neox=neox, rotary_dim=module.rotary_dim)


@pytest.mark.parametrize("D,neox,partial", [(128, True, 1.0), (128, False, 1.0), (64, True, 1.0), (64, False, 1.0),
                                            (128, True, 0.5), (64, False, 0.5), (128, False, 0.25),
                                            (256, False, 0.25), (256, True, 1.0), (96, True, 1.0), (96, False, 0.5)])
def test_dense_rope_is_bit_exact(device, D, neox, partial):
    B, Hq, Hk, S = 3, 8, 2, 19
    mod = _module(D, partial_rotary_factor=partial)
    g = torch.Generator().manual_seed(D + int(neox))
    pos = torch.randint(0, 512, (B, S), generator=g)
    q, k = seeded_q(1, B, Hq, S, D), seeded_q(2, B, Hk, S, D)
    rope = mod(q.to(device), pos.to(device))
    qo, ko = rope(q.to(device), k.to(device), is_neox_style=neox)
    assert_bits_equal(qo, _oracle_rotate(q, mod, pos, neox), "query")
    assert_bits_equal(ko, _oracle_rotate(k, mod, pos, neox), "key")


@pytest.mark.parametrize("D,neox,partial", [(128, True, 1.0), (80, False, 1.0), (64, True, 0.5), (20, True, 1.0), (256, False, 0.25)])
def test_dense_rope_on_fp32_tensors_is_bit_exact(device, D, neox, partial):
    """The reference's operator takes any float dtype (cos / sin are cast to it, :398-399); on fp32 every product
    and the sum are separate fp32 roundings."""
    B, Hq, Hk, S = 2, 4, 2, 11
    mod = _module(D, partial_rotary_factor=partial)
    g = torch.Generator().manual_seed(D)
    pos = torch.randint(0, 512, (B, S), generator=g)
    q, k = torch.randn(B, Hq, S, D, generator=g), torch.randn(B, Hk, S, D, generator=g)
    rope = mod(q.to(device), pos.to(device))
    qo, ko = rope(q.to(device), k.to(device), is_neox_style=neox)
    assert qo.dtype == torch.float32
    assert torch.equal(qo.cpu(), _oracle_rotate(q, mod, pos, neox)), "query"
    assert torch.equal(ko.cpu(), _oracle_rotate(k, mod, pos, neox)), "key"


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_rope_on_token_major_tensors_and_with_one_row_of_positions(device, dtype):
    """unsqueeze_dim=2 rotates [B, S, H, D] tensors (:418-419); position ids / cos of batch 1 serve every sequence,
    as cos.unsqueeze(1) broadcasts in the reference."""
    B, H, S, D = 3, 4, 7, 128
    mod = _module(D)
    g = torch.Generator().manual_seed(5)
    q = torch.randn(B, S, H, D, generator=g).to(dtype)
    k = torch.randn(B, S, 2, D, generator=g).to(dtype)
    pos = torch.arange(40, 40 + S).view(1, S)
    want_q = _oracle_rotate(q.transpose(1, 2), mod, pos.expand(B, S), True).transpose(1, 2)
    want_k = _oracle_rotate(k.transpose(1, 2), mod, pos.expand(B, S), True).transpose(1, 2)
    cos, sin = mod(q.to(device), pos.to(device), return_cos_sin=True)
    assert cos.shape[0] == 1
    qo, ko = mod.apply_rotary_emb(q.to(device), k.to(device), cos, sin, unsqueeze_dim=2)
    assert torch.equal(qo.cpu(), want_q) and torch.equal(ko.cpu(), want_k)
    rope = mod(q.to(device), pos.to(device))            # [1, S] rows kept by the callable as well
    qo2, _ = rope(q.to(device), None, unsqueeze_dim=2)
    assert torch.equal(qo2.cpu(), want_q)
    qo3, _ = rope(q.to(device).transpose(1, 2), None)   # the same rows as [B, H, S, D]
    assert torch.equal(qo3.cpu(), want_q.transpose(1, 2))
    with pytest.raises(RuntimeError, match="position rows"):
        mod(q.to(device), torch.zeros(2, S, dtype=torch.long, device=device))(q.to(device).transpose(1, 2), None)


def test_longrope_always_pairs_halves(device):
    """The reference's longrope branch never looks at is_neox_style (:421-430)."""
    D, S = 128, 9
    cfg = dict(rope_type="longrope", short_factor=[1.0 + 0.01 * i for i in range(D // 2)],
               long_factor=[2.0 + 0.02 * i for i in range(D // 2)])
    mod = _module(D, rows=256, scaling=cfg, original_max_position_embeddings=128)
    q = seeded_q(8, 2, 4, S, D)
    pos = torch.arange(S).repeat(2, 1)
    rope = mod(q.to(device), pos.to(device))
    a, _ = rope(q.to(device), None, is_neox_style=False)
    b, _ = rope(q.to(device), None, is_neox_style=True)
    assert_bits_equal(a, b, "is_neox_style ignored")
    cos, sin = rope_ref.lookup(mod.cos_cache, mod.sin_cache, rope_ref.longrope_rows(pos, 128), q.dtype)
    assert_bits_equal(a, rope_ref.rotate_longrope_form(q, cos, sin, D), "longrope form")


def test_dense_rope_takes_transposed_views_and_leaves_inputs_alone(device):
    """The models hand in [B, S, H, D] projections viewed as [B, H, S, D] (llama.py:125-138)."""
    B, H, S, D = 2, 4, 9, 128
    mod = _module(D)
    pos = torch.arange(100, 100 + S).repeat(B, 1)
    q = seeded_q(3, B, S, H, D)  # [B, S, H, D] storage
    qd = q.to(device)
    view = qd.transpose(1, 2)
    before = qd.clone()
    rope = mod(view, pos.to(device))
    qo, none = rope(view, None)
    assert none is None
    assert_bits_equal(qd, before, "input untouched")
    assert_bits_equal(qo, _oracle_rotate(q.transpose(1, 2), mod, pos), "rotated view")


def test_apply_rotary_emb_with_gathered_cos_sin(device):
    """Second calling convention of the reference operator (return_cos_sin=True, then apply_rotary_emb)."""
    B, Hq, Hk, S, D = 2, 4, 2, 6, 64
    mod = _module(D, scaling=dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                                  original_max_position_embeddings=128))
    pos = torch.tensor([[0, 1, 2, 3, 4, 5], [300, 301, 302, 303, 304, 305]])
    q, k = seeded_q(4, B, Hq, S, D), seeded_q(5, B, Hk, S, D)
    cos, sin = mod(q, pos, return_cos_sin=True)
    assert cos.dtype == torch.bfloat16 and cos.shape == (B, S, D // 2)
    qo, ko = mod.apply_rotary_emb(q.to(device), k.to(device), cos.to(device), sin.to(device))
    assert_bits_equal(qo, rope_ref.rotate(q, cos, sin), "query")
    assert_bits_equal(ko, rope_ref.rotate(k, cos, sin), "key")


def test_fp32_tables_are_rounded_like_the_reference(device):
    """pace_rope_t with fp32 tables: entries are rounded to bf16 on load (`.to(x.dtype)`)."""
    from pace_mi355 import _native as nat

    B, H, S, D = 1, 2, 5, 128
    mod = _module(D)
    pos = torch.tensor([[7, 8, 9, 400, 511]])
    q = seeded_q(6, B, H, S, D)
    qd = q.to(device)
    out = torch.empty_like(qd)
    cos32, sin32 = mod.cos_cache.to(device).contiguous(), mod.sin_cache.to(device).contiguous()
    rows = pos.to(device=device, dtype=torch.int32)
    d = nat.RopeDesc(cos=cos32.data_ptr(), sin=sin32.data_ptr(), table_dtype=nat.DTYPE_F32, table_rows=512, rotary_dim=D,
                     interleaved=0, positions=rows.data_ptr(), pos_stride_b=rows.stride(0))
    nat.check(nat.load().pace_rope_apply(ctypes.byref(d), qd.data_ptr(), out.data_ptr(), qd.stride(0), qd.stride(1), qd.stride(2), H,
                                         None, None, 0, 0, 0, 0, B, S, D, nat.current_stream_ptr()))
    assert_bits_equal(out, _oracle_rotate(q, mod, pos), "fp32 table")


@pytest.mark.parametrize("D,neox,steps", [(128, True, [5, 1, 1, 40, 1]), (64, False, [17, 3, 1]), (128, False, [1, 1, 16, 33]),
                                          (256, False, [5, 1, 16, 9]), (96, True, [5, 1, 16, 9])])
def test_rope_append_fills_the_pool_like_rope_then_update_cache(device, D, neox, steps):
    """rope(k) then update_cache (llama.py:147-158) == one rotate-and-append launch, bit for bit."""
    from pace_mi355.llm import PagedKVCache

    B, hkv, n_rep = 2, 2, 4
    mod = _module(D, rows=256)
    cache = PagedKVCache(256, num_kv_heads=hkv, n_rep=n_rep)
    cache.fuse_append = False  # every update launches pace_rope_append_paged at once
    ref = DynamicKVCacheRef(256)
    past = 0
    for i, T in enumerate(steps):
        k, v = seeded_kv(100 + i, B, hkv, T, D)
        pos = torch.arange(past, past + T).repeat(B, 1)
        rope = mod(k.to(device), pos.to(device)).with_style(neox)
        cache.update_cache(k.to(device), v.to(device), 2, rope=rope)
        ref.update_cache(_oracle_rotate(k, mod, pos, neox), v, 2)
        past += T
        kg, vg = cache.gather(n_rep=1)
        assert_bits_equal(kg, ref.key, f"K after step {i}")
        assert_bits_equal(vg, ref.value, f"V after step {i}")


def test_rope_append_rotates_queries_in_the_same_launch(device):
    """C ABI: q rotated into q_out while k/v go to the pool; positions derived from the lengths."""
    from pace_mi355 import _native as nat
    from pace_mi355.llm import PagedKVCache

    B, hkv, n_rep, D, T = 3, 2, 4, 128, 7
    lens0 = [20, 3, 40]
    mod = _module(D, rows=128)
    cache = PagedKVCache(128, num_kv_heads=hkv, n_rep=n_rep)
    cache.fuse_append = False
    k0, v0 = seeded_kv(1, B, hkv, 40, D)
    cache.append_ragged(k0.to(device), v0.to(device), lens0)
    k, v = seeded_kv(2, B, hkv, T, D)
    q = seeded_q(3, B, hkv * n_rep, T, D)
    kd, vd, qd = k.to(device), v.to(device), q.to(device)
    q_out = torch.empty_like(qd)
    st = cache.state
    new_lens = cache.lens + T
    st.ensure_capacity(new_lens)
    (lens_dev, bias), table = st.device_lens(new_lens), st.device_table()
    cos, sin = mod.device_tables(qd.device)
    d = nat.RopeDesc(cos=cos.data_ptr(), sin=sin.data_ptr(), table_dtype=nat.DTYPE_BF16, table_rows=cos.shape[0], rotary_dim=D,
                     interleaved=0, positions=None, pos_stride_b=0)
    nat.check(nat.load().pace_rope_append_paged(
        ctypes.byref(cache._desc), ctypes.byref(d), qd.data_ptr(), q_out.data_ptr(), qd.stride(0), qd.stride(1), qd.stride(2),
        hkv * n_rep, kd.data_ptr(), vd.data_ptr(), kd.stride(0), kd.stride(1), kd.stride(2), B, T, table.data_ptr(), table.stride(0),
        lens_dev.data_ptr(), bias - T, nat.current_stream_ptr()))
    cache.lens, cache.seq_len = new_lens, int(new_lens.max())
    pos = torch.tensor([[l + t for t in range(T)] for l in lens0])
    assert_bits_equal(q_out, _oracle_rotate(q, mod, pos), "q_out")
    kg, vg = cache.gather(n_rep=1)
    k_rot = _oracle_rotate(k, mod, pos)
    for b, l in enumerate(lens0):
        assert_bits_equal(kg[b, :, :l], k0[b, :, :l], f"old K of sequence {b}")
        assert_bits_equal(kg[b, :, l:l + T], k_rot[b], f"new K of sequence {b}")
        assert_bits_equal(vg[b, :, l:l + T], v[b], f"new V of sequence {b}")


def _reference_step(q, k, v, mod, pos, ref_cache, n_rep, neox=True):
    """rope -> repeat_kv -> update_cache -> attention, as LlamaAttention.forward orders it."""
    qr, kr = _oracle_rotate(q, mod, pos, neox), _oracle_rotate(k, mod, pos, neox)
    k_all, v_all = ref_cache.update_cache(kr, v, 2)
    L, S = k_all.shape[2], q.shape[2]
    mask = torch.zeros(1, 1, S, L)
    for s in range(S):
        mask[0, 0, s, L - S + s + 1:] = float("-inf")
    return sdpa_fp32(qr, repeat_kv(k_all, n_rep), repeat_kv(v_all, n_rep), mask)


@pytest.mark.parametrize("D,neox,S", [(128, True, 1), (128, False, 1), (64, True, 1), (128, True, 8), (64, False, 5), (128, True, 20),
                                      (256, True, 1), (256, False, 4), (96, True, 1), (96, False, 3)])
def test_one_launch_step_rope_append_attention(device, D, neox, S):
    """update_cache(raw k, v, rope) + attention(raw q): one launch per step; pool bit-exact,
    attention within tolerance, and identical to rotating in a launch of its own."""
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.ops import MultiHeadAttention

    B, hkv, n_rep, prompt, steps = 3, 2, 4, 70, 3
    mod = _module(D, rows=256)
    fused = PagedKVCache(256, num_kv_heads=hkv, n_rep=n_rep)
    split = PagedKVCache(256, num_kv_heads=hkv, n_rep=n_rep)
    ref = DynamicKVCacheRef(256)
    attn = MultiHeadAttention()
    past = 0
    for i, T in enumerate([prompt] + [S] * steps):
        k, v = seeded_kv(200 + i, B, hkv, T, D)
        q = seeded_q(300 + i, B, hkv * n_rep, T, D)
        pos = torch.arange(past, past + T).repeat(B, 1)
        kd, vd, qd = k.to(device), v.to(device), q.to(device)
        rope = mod(kd, pos.to(device)).with_style(neox)
        want = _reference_step(q, k, v, mod, pos, ref, n_rep, neox)
        # one launch (steps of <= 32 tokens) / rotate-and-append + attention (the prompt)
        kk, vv = fused.update_cache(kd, vd, 2, rope=rope)
        got = attn(qd, kk, vv)
        assert_attention_close(got, want, f"step {i} fused")
        # the rotation as its own launch, then the same append + attention launch without it:
        # the same arithmetic in the same order, so the outputs agree bit for bit
        q_rot, k_rot = rope(qd, kd)
        kk2, vv2 = split.update_cache(k_rot, vd, 2)
        got2 = attn(q_rot, kk2, vv2)
        # (head size 96 included: there the halves of a pair lie in lanes 32 apart, which exchange them in registers)
        assert_bits_equal(got, got2, f"step {i}: fused launch vs separate launches")
        past += T
        kg, vg = fused.gather(n_rep=1)
        assert_bits_equal(kg, ref.key, f"pool K after step {i}")
        assert_bits_equal(vg, ref.value, f"pool V after step {i}")


def test_rope_with_left_padded_positions_and_mask(device):
    """Left-padded batch as the reference runs it: position ids from the padding mask
    (llama.py:300-303) and an explicit additive mask; the rotation then runs as its own launch."""
    from oracle.attention_ref import causal_mask_4d
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.ops import MultiHeadAttention

    B, hkv, n_rep, D, L = 2, 2, 2, 128, 24
    pad = [0, 9]
    mask2d = torch.ones(B, L, dtype=torch.long)
    for b, p in enumerate(pad):
        mask2d[b, :p] = 0
    pos = mask2d.cumsum(-1) - 1
    pos.masked_fill_(mask2d == 0, 1)
    mod = _module(D, rows=64)
    k, v = seeded_kv(7, B, hkv, L, D)
    q = seeded_q(8, B, hkv * n_rep, L, D)
    mask4d = causal_mask_4d(mask2d, L, L, torch.bfloat16)
    cache = PagedKVCache(64, num_kv_heads=hkv, n_rep=n_rep)
    rope = mod(k.to(device), pos.to(device))
    kk, vv = cache.update_cache(k.to(device), v.to(device), 2, rope=rope)
    got = MultiHeadAttention()(q.to(device), kk, vv, attention_mask=mask4d.to(device))
    qr, kr = _oracle_rotate(q, mod, pos), _oracle_rotate(k, mod, pos)
    want = sdpa_fp32(qr, repeat_kv(kr, n_rep), repeat_kv(v, n_rep), mask4d)
    for b, p in enumerate(pad):  # rows of padding queries are unspecified in the reference as well
        assert_attention_close(got[b, :, p:], want[b, :, p:], f"sequence {b}")
    kg, _ = cache.gather(n_rep=1)
    assert_bits_equal(kg, kr, "pool K")


def test_longrope_rows_follow_the_reference_switch(device):
    short = [1.0 + 0.02 * i for i in range(32)]
    long_ = [3.0 + 0.1 * i for i in range(32)]
    mod = _module(64, rows=256, scaling=dict(rope_type="longrope", short_factor=short, long_factor=long_),
                  original_max_position_embeddings=64)
    assert mod.cos_cache.shape == (64 + 256, 32)
    B, H, S = 1, 2, 4
    q = seeded_q(9, B, H, S, 64)
    for pos in (torch.tensor([[10, 11, 12, 13]]), torch.tensor([[62, 63, 64, 65]])):
        rope = mod(q.to(device), pos.to(device))
        rows = rope_ref.longrope_rows(pos, 64)
        assert torch.equal(rope.rows.cpu().long(), rows)
        qo, _ = rope(q.to(device), None)
        cos, sin = rope_ref.lookup(mod.cos_cache, mod.sin_cache, rows, torch.bfloat16)
        assert_bits_equal(qo, rope_ref.rotate_longrope_form(q, cos, sin, 64), "longrope")


@pytest.mark.parametrize("neox,rot", [(True, 80), (False, 80), (True, 64)])
def test_rope_with_a_zero_padded_head_size(device, neox, rot):
    """Head sizes the kernels are not built for (80: OPT-2.7B's) are kept zero-padded in slabs of the next built size;
    the rotation then runs over the first rotary_dim dims of the padded rows in launches of its own (inside the
    attention launch it takes rotary_dim == the pool's head size).  Pool contents bit-exact, attention within tolerance."""
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.ops import MultiHeadAttention

    B, hkv, n_rep, D = 2, 2, 2, 80
    mod = _module(rot, rows=128)
    cache = PagedKVCache(128, num_kv_heads=hkv, n_rep=n_rep)
    ref = DynamicKVCacheRef(128)
    attn = MultiHeadAttention()
    past = 0
    for i, T in enumerate([37, 1, 3, 1]):
        k, v = seeded_kv(500 + i, B, hkv, T, D)
        q = seeded_q(600 + i, B, hkv * n_rep, T, D)
        pos = torch.arange(past, past + T).repeat(B, 1)
        kd, vd, qd = k.to(device), v.to(device), q.to(device)
        rope = mod(kd, pos.to(device)).with_style(neox)
        want = _reference_step(q, k, v, mod, pos, ref, n_rep, neox)
        kk, vv = cache.update_cache(kd, vd, 2, rope=rope)
        assert cache.head_dim == 96 and cache.model_dim == 80
        got = attn(qd, kk, vv)
        assert got.shape == q.shape
        assert_attention_close(got, want, f"step {i}")
        past += T
        kg, vg = cache.gather(n_rep=1)
        assert_bits_equal(kg, ref.key, f"pool K after step {i}")
        assert_bits_equal(vg, ref.value, f"pool V after step {i}")
