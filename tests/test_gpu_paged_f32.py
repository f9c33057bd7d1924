"""GPU parity of the paged cache with an fp32 pool (the reference's caches keep the model's dtype,
``pace/llm/cache.py:255-266``; its attention is registered for float32 and bfloat16,
``pace/ops/backends/jit.py:31-34``): storage bit-exact against the contiguous-semantics oracle,
attention within 1e-5 of the fp32 oracle."""
import ctypes

import numpy as np
import pytest
import torch

from helpers import assert_bits_equal, seeded_kv, seeded_q
from oracle.attention_ref import causal_mask_4d, sdpa_fp32
from oracle.cache_ref import DynamicKVCacheRef, repeat_kv, valid_prefix
from oracle.paged_ref import RaggedCacheModel

pytestmark = pytest.mark.gpu
F32 = torch.float32


def _paged(max_len, **kw):
    from pace_mi355.llm import PagedKVCache

    return PagedKVCache(max_len, **kw)


def _close(out, ref, what, atol=1e-5, rtol=1e-5):
    o, r = out.detach().cpu(), ref.detach().cpu()
    assert o.dtype == torch.float32 and o.shape == r.shape, f"{what}: {o.dtype} {tuple(o.shape)} vs {tuple(r.shape)}"
    assert not torch.isnan(o).any(), f"{what}: NaN in output"
    assert torch.allclose(o, r, atol=atol, rtol=rtol), f"{what}: max abs err {(o - r).abs().max().item():.3g}"


def _build(device, B, hkv, n_rep, D, lens, seed, num_blocks=None):
    T = max(max(lens), 1)
    cache = _paged(T + 64, num_kv_heads=hkv, n_rep=n_rep, num_blocks=num_blocks)
    model = RaggedCacheModel(B, hkv, D, dtype=F32)
    k, v = seeded_kv(seed, B, hkv, T, D, dtype=F32)
    cache.append_ragged(k.to(device), v.to(device), lens)
    model.append(k, v, lens)
    return cache, model


@pytest.mark.parametrize("hkv,n_rep,dim", [(8, 4, 128), (2, 1, 64), (4, 1, 256), (2, 4, 96), (2, 2, 80), (3, 2, 100), (2, 1, 50), (1, 1, 4)])
def test_append_matches_reference_dynamic_cache(device, hkv, n_rep, dim):
    """The stream of ``tests/test_gpu_paged_cache.py`` in fp32: gather(expand) equals the reference tensors bit for bit
    (head sizes that are no multiple of 4 are kept zero-padded)."""
    B = 3
    ref = DynamicKVCacheRef(256)
    cache = _paged(256, num_kv_heads=hkv, n_rep=n_rep)
    for step, T in enumerate([37, 1, 1, 16, 5, 1]):
        k, v = seeded_kv(100 + step, B, hkv, T, dim, dtype=F32)
        k_exp, v_exp = repeat_kv(k, n_rep), repeat_kv(v, n_rep)
        rk, rv = ref.update_cache(k_exp, v_exp, concat_dim=2)
        pk, pv = cache.update_cache(k_exp.to(device), v_exp.to(device), concat_dim=2)
        assert cache.seq_len == ref.seq_len and cache.pool.dtype == F32
        assert_bits_equal(pk.dense(), rk, f"K after step {step}")
        assert_bits_equal(pv.dense(), rv, f"V after step {step}")
    ref.remove_cache(7)
    cache.remove_cache(7)
    rk, rv = valid_prefix(ref)
    assert_bits_equal(cache.key.dense(), rk, "K after remove_cache")
    assert_bits_equal(cache.value.dense(), rv, "V after remove_cache")
    with pytest.raises(RuntimeError, match="the cache holds torch.float32"):
        cache.update_cache(k_exp.to(device).bfloat16(), v_exp.to(device).bfloat16(), concat_dim=2)


def test_append_from_transposed_views(device):
    B, H, T, D = 2, 4, 9, 128
    g = torch.Generator().manual_seed(7)
    base_k, base_v = torch.randn(B, T, H, D, generator=g), torch.randn(B, T, H, D, generator=g)
    cache = _paged(64)
    pk, pv = cache.update_cache(base_k.to(device).transpose(1, 2), base_v.to(device).transpose(1, 2), concat_dim=2)
    assert_bits_equal(pk.dense(), base_k.transpose(1, 2).contiguous(), "K")
    assert_bits_equal(pv.dense(), base_v.transpose(1, 2).contiguous(), "V")


def test_ragged_append_truncate_evict_compact_reorder(device):
    B, H, D = 5, 2, 128
    rng = np.random.default_rng(11)
    cache = _paged(400, num_blocks=160)
    model = RaggedCacheModel(B, H, D, dtype=F32)
    for step in range(6):
        T = int(rng.integers(1, 40))
        counts = rng.integers(0, T + 1, size=B)
        k, v = seeded_kv(200 + step, B, H, T, D, dtype=F32)
        cache.append_ragged(k.to(device), v.to(device), counts)
        model.append(k, v, counts)
        assert cache.lens.tolist() == model.seq_lens()

    def check(tag):
        K, V = model.dense()
        gk, gv = cache.gather()
        assert_bits_equal(gk, K, f"K {tag}")
        assert_bits_equal(gv, V, f"V {tag}")

    check("after ragged appends")
    rem = [int(rng.integers(0, min(9, n + 1))) for n in model.seq_lens()]
    cache.truncate(rem)
    model.truncate(rem)
    check("after truncate")
    for b in range(B):
        nb = (model.seq_lens()[b] + 15) // 16
        drop = sorted(rng.choice(nb, size=nb * 2 // 5, replace=False).tolist()) if nb else []
        cache.evict_blocks(b, drop)
        model.evict_blocks(b, drop, 16)
    check("after evict")
    moved = cache.compact()
    live = cache.state.live_block_count()
    used = np.concatenate([cache.state.table[b, : cache.state.n_blocks[b]] for b in range(B)])
    assert sorted(used.tolist()) == list(range(live)) and moved <= live
    check("after compact")
    # beams: sequences become copies of others, the shared tail blocks are copied when written
    order = [3, 3, 0, 1, 1]
    cache.reorder(order)
    model.reorder(order)
    check("after reorder")
    k, v = seeded_kv(300, B, H, 20, D, dtype=F32)
    cache.append_ragged(k.to(device), v.to(device), [20] * B)
    model.append(k, v)
    check("after the append that follows")
    assert cache.cow_blocks_copied > 0


@pytest.mark.parametrize("hkv,n_rep,dim", [(2, 1, 128), (8, 4, 128), (2, 2, 64), (1, 3, 256), (2, 1, 80), (2, 2, 36)])
def test_packed_gather_and_gather_without_zero_fill(device, hkv, n_rep, dim):
    B = 6
    lens = [0, 1, 16, 17, 333, 40]
    cache = _paged(400, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, dim, dtype=F32)
    k, v = seeded_kv(77, B, hkv, max(lens), dim, dtype=F32)
    cache.append_ragged(k.to(device), v.to(device), lens)
    model.append(k, v, lens)
    cache.truncate([0, 0, 3, 0, 13, 0])
    model.truncate([0, 0, 3, 0, 13, 0])
    lens = model.seq_lens()
    for rep in (1, n_rep):
        K, V = model.dense(rep)
        pk, pv, cu = cache.gather_packed(n_rep=rep)
        assert cu.cpu().tolist() == np.concatenate([[0], np.cumsum(lens)]).tolist()
        want_k = torch.cat([K[b, :, :n].transpose(0, 1) for b, n in enumerate(lens)], dim=0)
        want_v = torch.cat([V[b, :, :n].transpose(0, 1) for b, n in enumerate(lens)], dim=0)
        assert_bits_equal(pk, want_k, f"packed K n_rep={rep}")
        assert_bits_equal(pv, want_v, f"packed V n_rep={rep}")
        gk, gv = cache.gather(n_rep=rep, zero_fill=False)
        for b, n in enumerate(lens):
            assert_bits_equal(gk[b, :, :n], K[b, :, :n], f"K rows of sequence {b}")
            assert_bits_equal(gv[b, :, :n], V[b, :, :n], f"V rows of sequence {b}")
        gk, gv = cache.gather(n_rep=rep, pad_to=max(lens) + 5)
        Kp, Vp = model.dense(rep, pad_to=max(lens) + 5)
        assert_bits_equal(gk, Kp, "K zero-padded")
        assert_bits_equal(gv, Vp, "V zero-padded")


@pytest.mark.parametrize(
    "B,hkv,n_rep,D,lens",
    [
        (1, 1, 1, 128, [1]),
        (2, 2, 4, 128, [33, 64]),
        (4, 8, 4, 128, [64, 512, 100, 257]),
        (3, 2, 8, 128, [700, 31, 1500]),
        (2, 4, 1, 64, [129, 16]),
        (2, 1, 16, 128, [95, 300]),   # 16 query heads per KV head fill one row group
        (2, 1, 20, 128, [95, 300]),   # two row groups per KV head: the waves split the keys in two
        (2, 1, 40, 96, [95, 300]),    # three row groups: one wave each
        (3, 4, 1, 256, [700, 31, 1500]),
        (2, 2, 4, 256, [129, 4100]),
        (3, 4, 1, 80, [700, 31, 1500]),
        (2, 2, 2, 100, [5, 260]),     # a head size between two built ones
        (2, 2, 2, 50, [5, 260]),      # no multiple of 4: zero-padded
        (3, 2, 4, 128, [0, 1, 17]),   # an empty sequence gives zeros
    ],
)
def test_decode_matches_oracle(device, B, hkv, n_rep, D, lens):
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=B * 1000 + sum(lens))
    q = seeded_q(77, B, hkv * n_rep, 1, D, dtype=F32)
    out = cache.attend(q.to(device))
    ref = model.attention(q, n_rep)
    for b, n in enumerate(lens):
        if n == 0:
            assert (out[b] == 0).all(), "an empty sequence attends to nothing"
            ref[b] = 0
    _close(out, ref, f"decode lens={lens}")


@pytest.mark.parametrize("S,lens,n_rep,D", [(2, [40, 41], 4, 128), (8, [100, 8, 515], 4, 128), (16, [16, 33, 700], 1, 64),
                                             (20, [20, 333], 2, 128), (70, [70, 200], 4, 96), (130, [130, 400], 1, 256),
                                             (48, [48, 300], 2, 80), (33, [33, 100], 1, 100), (40, [77, 40, 1000], 4, 128)])
def test_verify_causal_matches_oracle(device, S, lens, n_rep, D):
    """S new tokens already appended; row s reads tokens <= len - S + s (``llama.py:292-299``)."""
    B, hkv = len(lens), 2
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=S * 31 + sum(lens))
    q = seeded_q(5, B, hkv * n_rep, S, D, dtype=F32)
    out = cache.attend(q.to(device))
    _close(out, model.attention(q, n_rep), f"verify S={S} lens={lens}")
    # the same through a strided view of the queries ([B, S, H, D] storage)
    qt = q.transpose(1, 2).contiguous().to(device).transpose(1, 2)
    assert_bits_equal(cache.attend(qt), out, "strided queries")


@pytest.mark.parametrize("S,n_rep,D", [(40, 2, 128), (70, 1, 80), (5, 4, 64)])
def test_kv_start_and_mask_tensors_with_many_query_rows(device, S, n_rep, D):
    """The launches whose workgroups share their tiles (more than 32 query rows per KV head), and a small one beside
    them: a first readable token per sequence, then an explicit mask tensor of each dtype with fewer columns than
    the longest sequence has tokens."""
    from oracle.attention_ref import lengths_mask_4d

    lens, hkv = [S + 3, 300, S + 130], 2
    B = len(lens)
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=S)
    q = seeded_q(4, B, hkv * n_rep, S, D, dtype=F32)
    K, V = model.dense(n_rep)
    start = torch.tensor([2, 37, 100], dtype=torch.int32)
    out = cache.attend(q.to(device), kv_start=start.to(device))
    _close(out, sdpa_fp32(q, K, V, lengths_mask_4d(lens, S, K.shape[2], F32, kv_start=start)), "kv_start")
    g = torch.Generator().manual_seed(S)
    for mdt in (torch.float32, torch.bfloat16):
        cols = 290
        m = torch.randn(B, 1, S, cols, generator=g).to(mdt)
        m[:, :, :, 17:40] = torch.finfo(mdt).min
        out = cache.attend(q.to(device), m.to(device))
        # the mask alone decides; a sequence's own length and the mask's width bound the columns
        full = torch.full((B, 1, S, K.shape[2]), float("-inf"))
        for b, n in enumerate(lens):
            full[b, :, :, : min(n, cols)] = m[b, :, :, : min(n, cols)].float()
        _close(out, sdpa_fp32(q, K, V, full), f"mask tensor {mdt}")


@pytest.mark.parametrize("mdt", [torch.float32, torch.bfloat16])
def test_additive_mask_path_matches_reference_semantics(device, mdt):
    """A left-padded batch the way the reference runs it (shared length, 4-D additive mask,
    ``llama.py:292-299``) through the attention operator; random masks; rows masked everywhere."""
    from pace_mi355.ops import MultiHeadAttention

    B, hkv, n_rep, D, L, S = 3, 2, 4, 128, 77, 1
    k, v = seeded_kv(9, B, hkv, L, D, dtype=F32)
    mask2d = torch.ones(B, L, dtype=torch.long)
    for b, p in enumerate([0, 13, 40]):
        mask2d[b, :p] = 0
    mask4d = causal_mask_4d(mask2d, S, L, mdt)
    cache = _paged(128, num_kv_heads=hkv, n_rep=n_rep)
    ke, ve = repeat_kv(k, n_rep), repeat_kv(v, n_rep)
    pk, pv = cache.update_cache(ke.to(device), ve.to(device), 2)
    q = seeded_q(10, B, hkv * n_rep, S, D, dtype=F32)
    mha = MultiHeadAttention(dtype=F32)
    out = mha(q.to(device), pk, pv, attention_mask=mask4d.to(device))
    _close(out, sdpa_fp32(q, ke, ve, mask4d), "masked decode")
    g = torch.Generator().manual_seed(3)
    rnd = torch.randn(1, 1, 1, L, generator=g).to(mdt)
    out = mha(q.to(device), pk, pv, attention_mask=rnd.to(device))
    _close(out, sdpa_fp32(q, ke, ve, rnd), "random additive mask")
    S2 = 6
    q2 = seeded_q(11, B, hkv * n_rep, S2, D, dtype=F32)
    m2 = causal_mask_4d(torch.ones(B, L, dtype=torch.long), S2, L, mdt)
    m2[1, :, :2, :] = torch.finfo(mdt).min
    out = mha(q2.to(device), pk, pv, attention_mask=m2.to(device))
    _close(out, sdpa_fp32(q2, ke, ve, m2), "rows masked everywhere")
    # a mask shorter than the sequences: the columns it does not have are masked
    short = torch.randn(B, 1, S2, 50, generator=g).to(mdt)
    out = cache.attend(q2.to(device), short.to(device))
    _close(out, sdpa_fp32(q2, ke[:, :, :50], ve[:, :, :50], short), "mask with fewer columns")
    # left padding as a start per sequence instead of a mask
    start = torch.tensor([0, 13, 40], dtype=torch.int32)
    out = cache.attend(q.to(device), kv_start=start.to(device))
    _close(out, sdpa_fp32(q, ke, ve, causal_mask_4d(mask2d, S, L, F32)), "kv_start")


def test_rope_rides_in_front_of_the_append_and_the_attention(device):
    from oracle import rope_ref
    from pace_mi355.ops import RotaryEmbedding

    B, hkv, n_rep, D = 3, 2, 4, 128
    mod = RotaryEmbedding(None, D, 256, 10000.0)
    cache = _paged(256, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, D, dtype=F32)
    past = 0
    for step, S in enumerate([40, 1, 1, 7]):
        k, v = seeded_kv(70 + step, B, hkv, S, D, dtype=F32)
        q = seeded_q(80 + step, B, hkv * n_rep, S, D, dtype=F32)
        pos = torch.arange(past, past + S).repeat(B, 1)
        rope = mod(k.to(device), pos.to(device))
        cos, sin = rope_ref.lookup(mod.cos_cache, mod.sin_cache, pos, F32)
        cache.update_cache(k.to(device), v.to(device), 2, rope=rope)
        model.append(rope_ref.rotate(k, cos, sin), v)
        out = cache.attend(q.to(device))
        _close(out, model.attention(rope_ref.rotate(q, cos, sin), n_rep), f"step {step}")
        past += S
    K, V = model.dense()
    gk, gv = cache.gather(n_rep=1)
    assert_bits_equal(gv, V, "V")
    _close(gk, K, "rotated K", atol=1e-6, rtol=1e-6)


def test_decode_invariant_to_physical_block_permutation(device):
    """The same tokens in differently numbered blocks give the same bits."""
    B, hkv, n_rep, D, lens = 3, 2, 4, 128, [200, 31, 333]
    a, _ = _build(device, B, hkv, n_rep, D, lens, seed=4, num_blocks=128)
    b = _paged(max(lens) + 64, num_kv_heads=hkv, n_rep=n_rep, num_blocks=128)
    k, v = seeded_kv(4, B, hkv, max(lens), D, dtype=F32)
    b.append_ragged(k[:, :, :1].to(device), v[:, :, :1].to(device), [0] * B)  # sets the state up, stores nothing
    rng = np.random.default_rng(0)
    ids = b.state.allocator.allocate(100)
    rng.shuffle(ids)
    b.state.allocator.free(ids)
    b.append_ragged(k.to(device), v.to(device), lens)
    assert not np.array_equal(a.state.table[:, :2], b.state.table[:, :2])
    q = seeded_q(1, B, hkv * n_rep, 3, D, dtype=F32).to(device)
    assert_bits_equal(a.attend(q), b.attend(q), "permuted blocks")


def _direct_args(cache, q, out, max_len):
    from pace_mi355 import _native as nat

    st = cache.state
    table, (lens_dev, bias) = st.device_table(), st.device_lens(cache.lens)
    a = nat.PagedAttnArgs()
    a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
    a.block_table, a.table_stride, a.seq_lens, a.seq_len_bias = table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias
    a.batch, a.num_q_heads, a.q_len, a.causal = q.shape[0], q.shape[1], q.shape[2], 1
    a.max_seq_len, a.scale = max_len, q.shape[3] ** -0.5
    return a, (table, lens_dev)


@pytest.mark.parametrize("S,n_rep,D,lens", [(1, 4, 128, [3000, 100]), (3, 4, 128, [3000, 100]), (1, 1, 64, [1029]), (9, 2, 256, [77, 2100, 0]),
                                             (40, 1, 96, [40, 1500])])
def test_sequences_cut_over_workgroups_when_a_workspace_is_given(device, S, n_rep, D, lens):
    """A batch that leaves compute units idle: with a workspace the launch cuts every sequence over several workgroups
    and merges; without one a workgroup walks its sequence alone.  Both match the oracle."""
    from pace_mi355 import _native as nat

    B, hkv = len(lens), 2
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=17 + S)
    q = seeded_q(3, B, hkv * n_rep, S, D, dtype=F32)
    ref = model.attention(q, n_rep)
    for b, n in enumerate(lens):
        if n == 0:
            ref[b] = 0
    qd = q.to(device)
    lib, stream = nat.load(), nat.current_stream_ptr()
    outs = []
    for ws_bytes in (0, 8 << 20, 100_000):  # none; room for every cut; room for a few
        out = torch.full_like(qd, float("nan"))
        a, keep = _direct_args(cache, qd, out, max(lens))
        ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device=device)
        if ws_bytes:
            a.workspace, a.workspace_bytes = ws.data_ptr(), ws_bytes
        fn = lib.pace_paged_attn_decode if S == 1 else lib.pace_paged_attn_verify
        nat.check(fn(ctypes.byref(cache._desc), ctypes.byref(a), stream))
        _close(out, ref, f"workspace of {ws_bytes} bytes")
        outs.append(out.cpu())
    assert not torch.equal(outs[0], outs[1]), "the cut was expected to change the order of the sums"
    assert_bits_equal(cache.attend(qd), outs[1], "PagedKVCache.attend passes a workspace for small batches")


def test_entry_points_that_fold_steps_in_refuse_an_fp32_pool(device):
    from pace_mi355 import _native as nat

    cache, _ = _build(device, 2, 2, 2, 128, [20, 5], seed=1)
    lib = nat.load()
    q = seeded_q(3, 2, 4, 1, 128, dtype=F32).to(device)
    out = torch.empty_like(q)
    a, (table, lens_dev) = _direct_args(cache, q, out, 20)
    bias = a.seq_len_bias
    stream = nat.current_stream_ptr()
    # the entry point that allocates nothing takes the pool too (this kernel has no scratch at all)
    nat.check(lib.pace_paged_attn_verify_static(ctypes.byref(cache._desc), ctypes.byref(a), stream))
    assert_bits_equal(out, cache.attend(q), "static entry point")
    # a rotary embedding never rides in the launch over an fp32 pool; a fused append only with up to 32 query rows per KV head
    rope = nat.RopeDesc()
    a.rope = ctypes.pointer(rope)
    assert lib.pace_paged_attn_decode(ctypes.byref(cache._desc), ctypes.byref(a), stream) != 0
    assert "fp32 pool" in lib.pace_kv_last_error().decode()
    a.rope = None
    S = 20  # 40 query rows per KV head
    q2 = seeded_q(4, 2, 4, S, 128, dtype=F32).to(device)
    out2 = torch.empty_like(q2)
    a2, keep = _direct_args(cache, q2, out2, 20)
    kn = torch.zeros(2, 2, S, 128, device=device)
    a2.k_new, a2.v_new, a2.n_new = kn.data_ptr(), kn.data_ptr(), S
    a2.new_stride_b, a2.new_stride_h, a2.new_stride_t = kn.stride(0), kn.stride(1), kn.stride(2)
    assert lib.pace_paged_attn_verify(ctypes.byref(cache._desc), ctypes.byref(a2), stream) != 0
    assert "up to 32 query rows" in lib.pace_kv_last_error().decode()
    k = torch.zeros(2, 2, 1, 128, dtype=torch.bfloat16, device=device)
    rc = lib.pace_rope_append_paged(ctypes.byref(cache._desc), ctypes.byref(nat.RopeDesc()), None, None, 0, 0, 0, 0, k.data_ptr(),
                                    k.data_ptr(), k.stride(0), k.stride(1), k.stride(2), 2, 1, table.data_ptr(), table.stride(0),
                                    lens_dev.data_ptr(), bias, stream)
    assert rc != 0 and "bf16 pools only" in lib.pace_kv_last_error().decode()


@pytest.mark.parametrize("T,n_rep,D,lens", [
    (1, 4, 128, [4096, 33, 1500, 15]),      # decode; a token that opens a block (15 -> 16) and ones that do not
    (1, 1, 64, [16, 31, 700]),              # no GQA; lengths on and next to block boundaries
    (4, 4, 128, [300, 14, 2000, 61, 5]),    # 16 query rows; new tokens straddling a block boundary (14 + 4, 61 + 4)
    (8, 4, 100, [1000, 9]),                 # 32 query rows, a head size that is none of the built ones
    (3, 8, 128, [40]),                      # one short sequence (cut over several workgroups through the workspace)
    (2, 2, 256, [500, 3000]),
])
def test_fused_append_equals_append_then_attend(device, T, n_rep, D, lens):
    """update_cache holds the new tokens back and the attention launch both reads them from the caller's tensors and
    stores them into the pool (launches of up to 32 query rows per KV head): the same attention result as
    append-then-attend, within 1e-5 of the oracle, and bit-identical pool contents; the step after reads the stored
    rows from the pool."""
    B, hkv = len(lens), 2
    k_new, v_new = seeded_kv(900 + T, B, hkv, T, D, dtype=F32)
    q = seeded_q(901, B, hkv * n_rep, T, D, dtype=F32)
    outs, caches = [], []
    for fuse in (True, False):
        cache, model = _build(device, B, hkv, n_rep, D, lens, seed=sum(lens) + T)
        cache.fuse_append = fuse
        cache.update_cache(repeat_kv(k_new, n_rep).to(device), repeat_kv(v_new, n_rep).to(device), 2)
        assert (cache._pending is not None) == fuse
        outs.append(cache.attend(q.to(device)))
        assert cache._pending is None
        caches.append(cache)
    model.append(k_new, v_new)
    ref = model.attention(q, n_rep)
    _close(outs[0], ref, "fused")
    _close(outs[1], ref, "unfused")
    K, V = model.dense(1)
    for c in caches:
        gk, gv = c.gather(n_rep=1)
        assert_bits_equal(gk, K, "pool K")
        assert_bits_equal(gv, V, "pool V")
    q1 = seeded_q(902, B, hkv * n_rep, 1, D, dtype=F32)
    k1, v1 = seeded_kv(903, B, hkv, 1, D, dtype=F32)
    caches[0].update_cache(k1.to(device), v1.to(device), 2)
    model.append(k1, v1)
    _close(caches[0].attend(q1.to(device)), model.attention(q1, n_rep), "step after the fused one")


def test_held_back_append_is_stored_first_when_the_launch_has_too_many_rows(device):
    """More than 32 query rows per KV head over an fp32 pool: the held-back append goes out as a launch of its own."""
    B, hkv, n_rep, D, T = 2, 2, 4, 128, 12   # 48 rows
    cache, model = _build(device, B, hkv, n_rep, D, [200, 70], seed=5)
    k_new, v_new = seeded_kv(7, B, hkv, T, D, dtype=F32)
    q = seeded_q(8, B, hkv * n_rep, T, D, dtype=F32)
    cache.update_cache(k_new.to(device), v_new.to(device), 2)
    assert cache._pending is not None
    out = cache.attend(q.to(device))
    model.append(k_new, v_new)
    _close(out, model.attention(q, n_rep), "48 rows")
    K, V = model.dense(1)
    gk, gv = cache.gather(n_rep=1)
    assert_bits_equal(gk, K, "pool K")
    assert_bits_equal(gv, V, "pool V")


@pytest.mark.parametrize("seed", range(6))
def test_random_histories(device, seed):
    """Appends, rollbacks, evictions, compactions and beam reorders in random order; after each, the
    gathered tensors equal the model's bit for bit and a decode / verify step matches the oracle."""
    rng = np.random.default_rng(1000 + seed)
    B, hkv, n_rep = int(rng.integers(1, 5)), int(rng.choice([1, 2, 4])), int(rng.choice([1, 2, 4]))
    D = int(rng.choice([64, 80, 128, 256]))
    cache = _paged(600, num_kv_heads=hkv, n_rep=n_rep, num_blocks=B * 40)
    model = RaggedCacheModel(B, hkv, D, dtype=F32)
    for step in range(14):
        op = rng.choice(["append", "append", "append", "truncate", "evict", "compact", "reorder"]) if step else "append"
        if op == "append":
            T = int(rng.integers(1, 48))
            room = [600 - n for n in model.seq_lens()]
            counts = [int(min(rng.integers(0, T + 1), r)) for r in room]
            k, v = seeded_kv(seed * 100 + step, B, hkv, T, D, dtype=F32)
            cache.append_ragged(k.to(device), v.to(device), counts)
            model.append(k, v, counts)
        elif op == "truncate":
            rem = [int(rng.integers(0, n + 1)) if n else 0 for n in model.seq_lens()]
            cache.truncate(rem)
            model.truncate(rem)
        elif op == "evict":
            b = int(rng.integers(0, B))
            nb = (model.seq_lens()[b] + 15) // 16
            drop = sorted(rng.choice(nb, size=nb // 3, replace=False).tolist()) if nb else []
            cache.evict_blocks(b, drop)
            model.evict_blocks(b, drop, 16)
        elif op == "compact":
            cache.compact()
        else:
            order = rng.integers(0, B, size=B).tolist()
            cache.reorder(order)
            model.reorder(order)
        assert cache.lens.tolist() == model.seq_lens()
        K, V = model.dense()
        gk, gv = cache.gather(n_rep=1)
        assert_bits_equal(gk, K, f"K after step {step} ({op})")
        assert_bits_equal(gv, V, f"V after step {step} ({op})")
        S = int(rng.choice([1, 1, 3]))
        if min(model.seq_lens()) >= S:
            q = seeded_q(step, B, hkv * n_rep, S, D, dtype=F32)
            _close(cache.attend(q.to(device)), model.attention(q, n_rep), f"attention after step {step} ({op})")


def test_manager_with_fp32_layers_and_beam_reorder(device):
    """The manager's call order of a model step (update per layer, attention, rollback, beam gather:
    ``pace/llm/cache.py:48-123``) with fp32 K/V; every layer shares the one block table."""
    from pace_mi355.llm import KVCacheManager, KVCacheType
    from pace_mi355.ops import MultiHeadAttention

    class Cfg:
        num_hidden_layers = 2
        num_attention_heads = 8
        num_key_value_heads = 2

    B = 3
    mgr = KVCacheManager(Cfg(), 96, KVCacheType.PAGED)
    refs = [DynamicKVCacheRef(96) for _ in range(2)]
    mha = MultiHeadAttention(dtype=F32)
    for step, T in enumerate([30, 1, 1, 5]):
        for layer in range(2):
            k, v = seeded_kv(400 + 10 * step + layer, B, 2, T, 128, dtype=F32)
            ke, ve = repeat_kv(k, 4), repeat_kv(v, 4)
            rk, rv = refs[layer].update_cache(ke, ve, 2)
            pk, pv = mgr[layer].update_cache(ke.to(device), ve.to(device), 2)
            q = seeded_q(500 + step, B, 8, T, 128, dtype=F32)
            L = refs[layer].seq_len
            mask = causal_mask_4d(torch.ones(B, L, dtype=torch.long), T, L, F32)
            out = mha(q.to(device), pk, pv, attention_mask=mask.to(device))
            _close(out, sdpa_fp32(q, rk, rv, mask), f"step {step} layer {layer}")
        assert len(mgr) == refs[0].seq_len
    mgr.remove_cache(3)
    beam = torch.tensor([2, 0, 0])
    mgr.update_cache_with_beam_indices(beam.to(device))
    for layer in range(2):
        refs[layer].remove_cache(3)
        refs[layer].update_cache_with_beam_indices(beam)
        rk, rv = valid_prefix(refs[layer])
        assert_bits_equal(mgr[layer].key.dense(), rk, f"layer {layer} K")
        assert_bits_equal(mgr[layer].value.dense(), rv, f"layer {layer} V")
    assert mgr[0].state is mgr[1].state and mgr[0].pool.dtype == F32


def test_decode_step_captured_into_a_graph(device):
    """``KVCacheManager.capture_decode`` with fp32 layers: per layer one launch (the append rides in the attention
    launch), captured once, replayed per token."""
    from pace_mi355.llm import KVCacheManager, KVCacheType
    from pace_mi355.ops import MultiHeadAttention

    class Cfg:
        num_hidden_layers = 2
        num_attention_heads = 8
        num_key_value_heads = 2

    B, hkv, n_rep, D, steps = 3, 2, 4, 128, 40
    lens0 = [300, 17, 1200]
    mgr = KVCacheManager(Cfg(), 2048, KVCacheType.PAGED)
    models = [RaggedCacheModel(B, hkv, D, dtype=F32) for _ in range(2)]
    for layer in range(2):
        k, v = seeded_kv(10 + layer, B, hkv, max(lens0), D, dtype=F32)
        mgr[layer].append_ragged(k.to(device), v.to(device), lens0)
        models[layer].append(k, v, lens0)
    mha = MultiHeadAttention(dtype=F32)
    qs = [torch.zeros(B, hkv * n_rep, 1, D, device=device) for _ in range(2)]
    ks = [torch.zeros(B, hkv, 1, D, device=device) for _ in range(2)]
    vs = [torch.zeros(B, hkv, 1, D, device=device) for _ in range(2)]

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
            kn, vn = seeded_kv(1000 + 2 * i + layer, B, hkv, 1, D, dtype=F32)
            qn = seeded_q(2000 + 2 * i + layer, B, hkv * n_rep, 1, D, dtype=F32)
            ks[layer].copy_(kn), vs[layer].copy_(vn), qs[layer].copy_(qn)
            models[layer].append(kn, vn)
            new.append(qn)
        outs = graph.replay()
        assert len(mgr) == max(lens0) + i + 1
        if i % 7 == 0 or i == steps - 1:
            for layer in range(2):
                _close(outs[layer], models[layer].attention(new[layer], n_rep), f"replay {i} layer {layer}")
    with pytest.raises(RuntimeError, match="reserved blocks for"):
        graph.replay()
    for layer in range(2):
        K, V = models[layer].dense(1)
        gk, gv = mgr[layer].gather(n_rep=1)
        assert_bits_equal(gk, K, f"pool K of layer {layer}")
        assert_bits_equal(gv, V, f"pool V of layer {layer}")
    # a second graph, ended early by a rollback; step-by-step operation carries on from there
    graph = mgr.capture_decode(step, max_steps=8)
    for layer in range(2):
        kn, vn = seeded_kv(5000 + layer, B, hkv, 1, D, dtype=F32)
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
        _close(outs[layer], models[layer].attention(qs[layer].cpu(), n_rep), f"eager step after the graph, layer {layer}")
