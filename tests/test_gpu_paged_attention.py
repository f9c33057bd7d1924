"""GPU parity: paged decode / verify attention against the fp32 oracle."""
import numpy as np
import pytest
import torch

from helpers import assert_attention_close, seeded_kv, seeded_q
from oracle.attention_ref import causal_mask_4d, lengths_mask_4d, sdpa_fp32
from oracle.cache_ref import repeat_kv
from oracle.paged_ref import RaggedCacheModel

pytestmark = pytest.mark.gpu


def _build(device, B, hkv, n_rep, D, lens, seed, partition=0, num_blocks=None, shuffle=True):
    from pace_mi355.llm import PagedKVCache

    T = max(lens)
    cache = PagedKVCache(T + 64, num_kv_heads=hkv, n_rep=n_rep, num_blocks=num_blocks)
    cache.partition_tokens = partition
    model = RaggedCacheModel(B, hkv, D)
    k, v = seeded_kv(seed, B, hkv, T, D)
    cache.append_ragged(k.to(device), v.to(device), lens)
    model.append(k, v, lens)
    return cache, model


@pytest.mark.parametrize(
    "B,hkv,n_rep,D,lens,partition",
    [
        (1, 1, 1, 128, [1], 0),
        (2, 2, 4, 128, [33, 64], 0),
        (4, 8, 4, 128, [64, 512, 100, 257], 0),       # plumbing shape (config 1 range)
        (3, 2, 8, 128, [700, 31, 1500], 256),         # several partitions + merge, 70B-style group of 8
        (2, 4, 1, 64, [129, 16], 128),                # head_dim 64, MHA
        (2, 1, 16, 128, [95, 300], 128),              # 16 query heads per KV head fill one tile
        (2, 1, 20, 128, [95, 300], 128),              # more than one query tile per KV head
        (3, 4, 1, 256, [700, 31, 1500], 256),         # head_dim 256 (GPT-J's heads), MHA, several partitions
        (2, 2, 4, 256, [129, 4100], 0),               # head_dim 256 with a GQA group
        (2, 1, 20, 256, [95, 300], 128),              # head_dim 256, two query tiles
        (3, 4, 1, 96, [700, 31, 1500], 256),          # head_dim 96 (Phi-3-mini's heads), several partitions
        (2, 2, 4, 96, [129, 4100], 0),                # head_dim 96 with a GQA group
        (2, 1, 40, 96, [95, 300], 128),               # head_dim 96, three query tiles
        (3, 4, 1, 80, [700, 31, 1500], 256),          # head_dim 80 (OPT-2.7B's heads): kept zero-padded in slabs of 96
    ],
)
def test_decode_matches_oracle(device, B, hkv, n_rep, D, lens, partition):
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=B * 1000 + sum(lens), partition=partition)
    q = seeded_q(77, B, hkv * n_rep, 1, D)
    out = cache.attend(q.to(device))
    ref = model.attention(q, n_rep)
    assert_attention_close(out, ref, f"decode lens={lens}")


@pytest.mark.parametrize("listed", [True, False])
def test_partitions_longer_than_one_fetch_of_block_ids(device, listed):
    """A wave holds the pool block ids of 64 of its units and fetches the next ones when it gets there: one
    partition of 20 000 tokens is 157 units per wave.  Through the planner's work list, and through the plain
    grid of a caller that passes no list."""
    import ctypes
    import math

    from pace_mi355 import _native as nat

    B, hkv, n_rep, D, lens = 2, 1, 4, 128, [20000, 9000]
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=99, partition=32768)
    q = seeded_q(7, B, hkv * n_rep, 1, D)
    ref = model.attention(q, n_rep)
    if listed:
        out = cache.attend(q.to(device))
    else:
        qd = q.to(device)
        out = torch.zeros_like(qd)
        st = cache.state
        table, (lens_dev, bias) = st.device_table(), st.device_lens(cache.lens)
        a = nat.PagedAttnArgs()
        a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = qd.data_ptr(), qd.stride(0), qd.stride(1), qd.stride(2)
        a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = out.data_ptr(), out.stride(0), out.stride(1), out.stride(2)
        a.block_table, a.table_stride, a.seq_lens, a.seq_len_bias = table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias
        a.causal, a.batch, a.num_q_heads, a.q_len = 1, B, hkv * n_rep, 1
        a.max_seq_len, a.partition_tokens, a.scale = max(lens), 32768, 1.0 / math.sqrt(D)
        nat.check(nat.load().pace_paged_attn_decode(ctypes.byref(cache._desc), ctypes.byref(a), nat.current_stream_ptr()))
    assert_attention_close(out, ref, "20 000-token partition")


def test_decode_empty_sequence_gives_zero(device):
    cache, model = _build(device, 2, 2, 2, 128, [0, 40], seed=3)
    q = seeded_q(1, 2, 4, 1, 128)
    out = cache.attend(q.to(device)).cpu().float()
    assert torch.count_nonzero(out[0]) == 0
    ref = model.attention(q, 2)
    assert_attention_close(out[1:], ref[1:], "non-empty row")


@pytest.mark.parametrize("S,lens,partition", [(8, [40, 200, 1029], 256), (9, [9, 64], 0), (3, [5, 300], 128), (16, [16, 100], 0),
                                               (40, [40, 333], 0), (130, [130, 700, 257], 256)])
def test_verify_causal_matches_oracle(device, S, lens, partition):
    """S new tokens already appended; row s reads tokens <= len - S + s (llama.py:292-299)."""
    B, hkv, n_rep, D = len(lens), 2, 4, 128
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=S * 31 + sum(lens), partition=partition)
    q = seeded_q(5, B, hkv * n_rep, S, D)
    out = cache.attend(q.to(device))
    ref = model.attention(q, n_rep)
    assert_attention_close(out, ref, f"verify S={S} lens={lens}")


def test_additive_mask_path_matches_reference_semantics(device):
    """Left-padded batch as the reference runs it: shared length, 2-D padding mask turned into
    the 4-D additive mask (llama.py:292-299) and handed to the attention operator."""
    from pace_mi355.ops import MultiHeadAttention

    B, hkv, n_rep, D, L, S = 3, 2, 4, 128, 77, 1
    k, v = seeded_kv(9, B, hkv, L, D)
    pad = [0, 13, 40]
    mask2d = torch.ones(B, L, dtype=torch.long)
    for b, p in enumerate(pad):
        mask2d[b, :p] = 0
    mask4d = causal_mask_4d(mask2d, S, L, torch.bfloat16)
    from pace_mi355.llm import PagedKVCache

    cache = PagedKVCache(128, num_kv_heads=hkv, n_rep=n_rep)
    ke, ve = repeat_kv(k, n_rep), repeat_kv(v, n_rep)
    pk, pv = cache.update_cache(ke.to(device), ve.to(device), 2)
    q = seeded_q(10, B, hkv * n_rep, S, D)
    mha = MultiHeadAttention(dtype=torch.bfloat16)
    out = mha(q.to(device), pk, pv, attention_mask=mask4d.to(device))
    ref = sdpa_fp32(q, ke, ve, mask4d)
    assert_attention_close(out, ref, "masked decode")
    # arbitrary (random) additive mask, fp32, broadcast over batch
    g = torch.Generator().manual_seed(3)
    rnd = torch.randn(1, 1, 1, L, generator=g)
    out = mha(q.to(device), pk, pv, attention_mask=rnd.to(device))
    assert_attention_close(out, sdpa_fp32(q, ke, ve, rnd), "random additive mask")
    # multi-token step whose first rows see nothing but finfo.min (pad positions of a left-padded
    # prompt): the reference's softmax makes them the plain average of V
    S2 = 6
    q2 = seeded_q(11, B, hkv * n_rep, S2, D)
    m2 = causal_mask_4d(torch.ones(B, L, dtype=torch.long), S2, L, torch.bfloat16)
    m2[1, :, :2, :] = torch.finfo(torch.bfloat16).min
    out = mha(q2.to(device), pk, pv, attention_mask=m2.to(device))
    assert_attention_close(out, sdpa_fp32(q2, ke, ve, m2), "rows masked everywhere")


@pytest.mark.parametrize("L,mdt", [(160, torch.bfloat16), (160, torch.float32), (157, torch.bfloat16), (157, torch.float32)])
@pytest.mark.parametrize("S", [1, 5, 12])
def test_mask_forms_partitions_and_fused_append(device, L, mdt, S):
    """Explicit masks through every way the kernel fetches them: whole 16-byte lines (length a multiple
    of 8) or element by element, bf16 or fp32, with the context cut into several partitions, with two
    query tiles per wave (12 tokens x 4 heads), and with the step's new tokens still held back, i.e.
    read from the caller's tensors at a position that is no multiple of 8."""
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.ops import MultiHeadAttention

    B, hkv, n_rep, D = 2, 2, 4, 128
    past = L - S
    k, v = seeded_kv(31, B, hkv, L, D)
    q = seeded_q(32, B, hkv * n_rep, S, D)
    m = causal_mask_4d(torch.ones(B, L, dtype=torch.long), S, L, mdt)
    m[0, :, :, :9] = torch.finfo(mdt).min                      # a left-padded row of the batch
    m = m + (torch.randn(B, 1, S, L, generator=torch.Generator().manual_seed(33)).to(mdt)) * (m == 0)
    ref = sdpa_fp32(q, repeat_kv(k, n_rep), repeat_kv(v, n_rep), m)
    mha = MultiHeadAttention(dtype=torch.bfloat16)
    for fuse in (True, False):
        cache = PagedKVCache(256, num_kv_heads=hkv, n_rep=n_rep)
        cache.partition_tokens = 64
        cache.fuse_append = fuse
        cache.update_cache(k[:, :, :past].to(device), v[:, :, :past].to(device), 2)
        cache.attend(seeded_q(34, B, hkv * n_rep, 1, D).to(device))  # flushes the prefill
        pk, pv = cache.update_cache(k[:, :, past:].to(device), v[:, :, past:].to(device), 2)
        assert (cache._pending is not None) == fuse
        out = mha(q.to(device), pk, pv, attention_mask=m.to(device))
        assert_attention_close(out, ref, f"L={L} {mdt} S={S} fused={fuse}")


@pytest.mark.parametrize("kind", ["causal", "left-padded", "row-masked-everywhere", "window", "real-only-past-the-end"])
def test_prefill_sized_masked_launch_leaves_out_only_what_weighs_nothing(device, kind):
    """More than 64 query rows per KV head with an explicit mask: the kernel looks over the mask and
    does not walk the units at the end of a wave's share that it rules out -- unless a row has no
    readable real value anywhere (it must end as the average of V).  Results must not depend on it."""
    from pace_mi355.llm import PagedKVCache

    B, hkv, n_rep, D, L, S = 2, 2, 4, 128, 700, 300
    k, v = seeded_kv(41, B, hkv, L, D)
    q = seeded_q(42, B, hkv * n_rep, S, D)
    dt = torch.bfloat16
    m = causal_mask_4d(torch.ones(B, L, dtype=torch.long), S, L, dt)
    cols = torch.arange(L)
    Lm = L
    if kind == "left-padded":
        m[1, :, :, :150] = torch.finfo(dt).min           # 150 pad columns: the forward look has to go past them
    elif kind == "row-masked-everywhere":
        m[0, :, 17, :] = torch.finfo(dt).min             # one row with nothing to read: nothing may be left out around it
    elif kind == "window":                               # sliding window: masked units on both sides of a band
        rows = torch.arange(S)[:, None] + (L - S)
        m = torch.zeros(B, 1, S, L, dtype=dt).masked_fill((cols[None, :] > rows) | (cols[None, :] < rows - 100), torch.finfo(dt).min)
    elif kind == "real-only-past-the-end":               # mask wider than the cache: zeros beyond the sequence must not count
        Lm = L + 64
        wide = torch.full((B, 1, S, Lm), torch.finfo(dt).min, dtype=dt)
        wide[..., :L] = m
        wide[0, :, 5, :] = torch.finfo(dt).min
        wide[0, :, 5, L:] = 0.0                           # row 5 of sequence 0 reads nothing it has: average of V
        m = wide
    bias = torch.randn(B, 1, S, Lm, generator=torch.Generator().manual_seed(43)).to(dt)
    m = m + bias * (m == 0)
    ref = sdpa_fp32(q, repeat_kv(k, n_rep), repeat_kv(v, n_rep), m[..., :L].contiguous())
    for partition in (0, 128):
        cache = PagedKVCache(L + 64, num_kv_heads=hkv, n_rep=n_rep)
        cache.partition_tokens = partition
        cache.update_cache(k.to(device), v.to(device), 2)
        out = cache.attend(q.to(device), m.to(device))
        assert_attention_close(out, ref, f"{kind} partition={partition}")


def test_masked_prefill_without_room_for_the_mask_summary(device):
    """The per-row mask summary is optional: a workspace without room for it (here: none at all) makes
    the launch walk every column, with the same result."""
    from pace_mi355.llm import PagedKVCache

    B, hkv, n_rep, D, L, S = 2, 2, 4, 128, 400, 200
    k, v = seeded_kv(51, B, hkv, L, D)
    q = seeded_q(52, B, hkv * n_rep, S, D)
    m = causal_mask_4d(torch.ones(B, L, dtype=torch.long), S, L, torch.bfloat16)
    ref = sdpa_fp32(q, repeat_kv(k, n_rep), repeat_kv(v, n_rep), m)
    cache = PagedKVCache(L + 64, num_kv_heads=hkv, n_rep=n_rep)
    cache.partition_tokens = 1024  # one partition per sequence: the partials need no workspace
    cache.update_cache(k.to(device), v.to(device), 2)
    with_summary = cache.attend(q.to(device), m.to(device))
    plan = cache.state.plan_attention
    cache.state.plan_attention = lambda *a: plan(*a)[:4] + (0,)  # same cut, no workspace
    without = cache.attend(q.to(device), m.to(device))
    assert_attention_close(with_summary, ref, "with the summary")
    assert_attention_close(without, ref, "without the summary")


def test_decode_invariant_to_physical_block_permutation(device):
    """Same logical cache, different physical block ids (via free-list history) -> same bits out."""
    B, hkv, n_rep, D, lens = 2, 2, 4, 128, [300, 123]
    q = seeded_q(4, B, hkv * n_rep, 1, D).to(device)
    cache_a, _ = _build(device, B, hkv, n_rep, D, lens, seed=21)
    out_a = cache_a.attend(q)
    from pace_mi355.llm import PagedKVCache

    cache_b = PagedKVCache(max(lens) + 64, num_kv_heads=hkv, n_rep=n_rep, num_blocks=200)
    # scramble the free list before use
    junk = cache_b  # allocate / free through the state once it exists
    k, v = seeded_kv(21, B, hkv, max(lens), D)
    cache_b.append_ragged(k[:, :, :1].to(device), v[:, :, :1].to(device), [0, 0])
    st = cache_b.state
    rng = np.random.default_rng(0)
    ids = st.allocator.allocate(150)
    rng.shuffle(ids)
    st.allocator.free(ids)
    cache_b.append_ragged(k.to(device), v.to(device), lens)
    assert not np.array_equal(cache_a.state.table[:, :5], cache_b.state.table[:, :5])
    out_b = cache_b.attend(q)
    assert torch.equal(out_a.cpu().view(torch.int16), out_b.cpu().view(torch.int16))


@pytest.mark.parametrize("T,S,lens,partition,D", [(1, 1, [40, 200, 1029, 16], 0, 128), (1, 1, [4096, 17], 512, 128),
                                                  (8, 8, [31, 700], 256, 128), (9, 9, [100, 64], 0, 128), (16, 1, [5, 48], 0, 128),
                                                  (32, 32, [33, 500], 0, 128), (1, 1, [40, 200, 1029, 16], 0, 256),
                                                  (5, 5, [31, 700], 256, 256), (1, 1, [77, 130], 0, 64),
                                                  (1, 1, [77, 1300], 0, 96), (7, 7, [40, 600], 256, 96), (1, 1, [77, 300], 0, 80)])
def test_fused_append_equals_append_then_attend(device, T, S, lens, partition, D):
    """update_cache holds the new tokens back and the attention launch both reads them from the
    caller's tensors and stores them: same attention result as append-then-attend (to tolerance, the
    summation order differs) and bit-identical cache contents."""
    B, hkv, n_rep = len(lens), 2, 4
    outs, caches = [], []
    k_new, v_new = seeded_kv(900 + T, B, hkv, T, D)
    q = seeded_q(901, B, hkv * n_rep, S, D)
    for fuse in (True, False):
        cache, model = _build(device, B, hkv, n_rep, D, lens, seed=sum(lens) + T, partition=partition)
        cache.fuse_append = fuse
        pk, pv = cache.update_cache(repeat_kv(k_new, n_rep).to(device), repeat_kv(v_new, n_rep).to(device), 2)
        assert (cache._pending is not None) == fuse
        outs.append(cache.attend(q.to(device)))
        assert cache._pending is None
        caches.append(cache)
    model.append(k_new, v_new)
    ref = model.attention(q, n_rep)
    assert_attention_close(outs[0], ref, "fused")
    assert_attention_close(outs[1], ref, "unfused")
    for c in caches:
        gk, gv = c.gather()
        K, V = model.dense(n_rep)
        assert torch.equal(gk.cpu(), K) and torch.equal(gv.cpu(), V)
    # the step after a fused one reads the stored tokens from the pool
    q1 = seeded_q(902, B, hkv * n_rep, 1, D)
    k1, v1 = seeded_kv(903, B, hkv, 1, D)
    caches[0].update_cache(k1.to(device), v1.to(device), 2)
    model.append(k1, v1)
    assert_attention_close(caches[0].attend(q1.to(device)), model.attention(q1, n_rep), "step after fused")


def test_pending_append_is_flushed_by_other_operations(device):
    cache, model = _build(device, 2, 2, 2, 128, [20, 37], seed=8)
    k1, v1 = seeded_kv(1, 2, 2, 1, 128)
    cache.update_cache(k1.to(device), v1.to(device), 2)
    model.append(k1, v1)
    assert cache._pending is not None
    cache.update_cache(k1.to(device), v1.to(device), 2)  # a second append flushes the first
    model.append(k1, v1)
    cache.truncate([1, 0])  # flushes the second
    model.truncate([1, 0])
    assert cache._pending is None
    K, V = model.dense(2)
    gk, gv = cache.gather()
    assert torch.equal(gk.cpu(), K) and torch.equal(gv.cpu(), V)


def test_chunked_prefill_through_the_paged_path(device):
    """A prompt fed in chunks: each chunk is appended and attends causally to everything so far
    (more query rows than one workgroup holds, several row groups per KV head)."""
    B, hkv, n_rep, D = 2, 2, 4, 128
    from pace_mi355.llm import PagedKVCache
    from oracle.paged_ref import RaggedCacheModel

    cache = PagedKVCache(512, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, D)
    for step, T in enumerate([100, 33, 64, 7]):
        k, v = seeded_kv(50 + step, B, hkv, T, D)
        q = seeded_q(60 + step, B, hkv * n_rep, T, D)
        pk, pv = cache.update_cache(k.to(device), v.to(device), 2)
        model.append(k, v)
        out = cache.attend(q.to(device))
        assert_attention_close(out, model.attention(q, n_rep), f"chunk {step} of {T} tokens")
    gk, gv = cache.gather()
    K, V = model.dense(n_rep)
    assert torch.equal(gk.cpu(), K) and torch.equal(gv.cpu(), V)


@pytest.mark.parametrize("T", [1, 5, 32])
def test_first_step_on_an_empty_cache(device, T):
    """The very first update: nothing is cached yet, the attention launch sees only the tokens it
    stores itself (fused) -- same as the reference's first update_cache + attention."""
    from pace_mi355.llm import PagedKVCache
    from oracle.paged_ref import RaggedCacheModel

    B, hkv, n_rep, D = 3, 2, 4, 128
    cache = PagedKVCache(128, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, D)
    for step in range(3):
        k, v = seeded_kv(40 + step, B, hkv, T, D)
        q = seeded_q(50 + step, B, hkv * n_rep, T, D)
        cache.update_cache(k.to(device), v.to(device), 2)
        assert cache._pending is not None
        model.append(k, v)
        out = cache.attend(q.to(device))
        assert_attention_close(out, model.attention(q, n_rep), f"T={T} step {step}")
    gk, gv = cache.gather(n_rep=1)
    K, V = model.dense(1)
    assert torch.equal(gk.cpu(), K) and torch.equal(gv.cpu(), V)


def test_fused_append_with_sequences_of_length_zero_and_one(device):
    """Ragged batch where some sequences hold nothing before the step."""
    cache, model = _build(device, 4, 2, 4, 128, [0, 1, 15, 16], seed=77)
    k1, v1 = seeded_kv(78, 4, 2, 1, 128)
    q = seeded_q(79, 4, 8, 1, 128)
    cache.update_cache(k1.to(device), v1.to(device), 2)
    model.append(k1, v1)
    out = cache.attend(q.to(device))
    assert_attention_close(out, model.attention(q, 4), "lens 0/1/15/16 + 1")
    # a sequence of one token attends to exactly that token: out == v
    torch.testing.assert_close(out[0].float().cpu(), repeat_kv(v1, 4)[0].float(), atol=1e-2, rtol=1e-2)
    gk, gv = cache.gather(n_rep=1)
    K, V = model.dense(1)
    assert torch.equal(gk.cpu(), K) and torch.equal(gv.cpu(), V)


@pytest.mark.parametrize("D,S,n_rep", [(128, 64, 4), (64, 48, 4), (128, 33, 8), (256, 24, 2), (96, 40, 4)])
def test_prefill_sized_launch_matches_oracle(device, D, S, n_rep):
    """A prefill-sized launch (hundreds of query rows per KV head over the whole batch): ragged
    lengths, a partly filled last row group, and a chunk appended on top of cached tokens."""
    B, hkv = 16, 8
    rng = np.random.default_rng(S)
    lens = (rng.integers(0, 300, B) + S).tolist()   # cached tokens + the S new ones
    lens[0], lens[1] = S, S + 1                    # nothing / one token cached before the chunk
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=S + D)
    q = seeded_q(31, B, hkv * n_rep, S, D)
    out = cache.attend(q.to(device))
    ref = model.attention(q, n_rep)
    assert_attention_close(out, ref, f"prefill-sized S={S} D={D}")


def _kernel_of(cache, q, lens, mask=None):
    """Name of the kernel an unfused attention call of this shape launches."""
    import math

    from pace_mi355 import _native as nat

    B, hq, S, D = q.shape
    table = cache.state.device_table()
    a = nat.PagedAttnArgs()
    a.q, a.q_stride_b, a.q_stride_h, a.q_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    a.out, a.o_stride_b, a.o_stride_h, a.o_stride_s = q.data_ptr(), q.stride(0), q.stride(1), q.stride(2)
    lens_dev = torch.tensor(lens, dtype=torch.int32, device=q.device)
    a.block_table, a.table_stride, a.seq_lens = table.data_ptr(), table.stride(0), lens_dev.data_ptr()
    a.causal, a.batch, a.num_q_heads, a.q_len = 1, B, hq, S
    a.max_seq_len, a.partition_tokens, a.scale = max(lens), 0, 1.0 / math.sqrt(D)
    if mask is not None:
        a.causal, a.mask, a.mask_dtype, a.mask_len = 0, mask.data_ptr(), nat.DTYPE_BF16, mask.size(3)
        a.mask_stride_b, a.mask_stride_s = mask.stride(0), mask.stride(2)
    return nat.kernel_name(cache._desc, a)


@pytest.mark.parametrize("D,S,n_rep,top", [(128, 64, 4, 2400), (64, 96, 4, 700)])
def test_cooperative_prefill_kernel_long_ragged_and_windowed(device, D, S, n_rep, top):
    """The workgroup-cooperative prefill kernel: ragged lengths past 64 units (the block ids are fetched 64
    units at a time), a row group that is only partly filled, and a first readable token per sequence
    (kv_start: aligned to a unit, inside one, zero, and past the chunk's first row)."""
    B, hkv = 16, 8
    rng = np.random.default_rng(D + S)
    lens = (rng.integers(S, top, B)).tolist()
    lens[0], lens[1], lens[2] = top, S, S + 31
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=S + D + 1)
    q = seeded_q(33, B, hkv * n_rep, S, D)
    qd = q.to(device)
    assert "paged_prefill_kernel" in _kernel_of(cache, qd, lens), "the case is meant for the cooperative kernel"
    starts = rng.integers(0, 200, B).astype(np.int32)
    starts[0], starts[1], starts[2], starts[3] = 0, 0, 64, 45
    starts = np.minimum(starts, np.array(lens, dtype=np.int32) - 1)
    for start in (None, starts):
        dev_start = None if start is None else torch.from_numpy(start).to(device)
        out = cache.attend(qd, kv_start=dev_start)
        K, V = model.dense(n_rep)
        mask = lengths_mask_4d(lens, S, K.shape[2], torch.float32, kv_start=start)
        ref = sdpa_fp32(q, K, V, mask)
        # a row whose window holds no token (start past its position) has no defined result in the oracle (it
        # averages every column); the kernels give 0 there
        empty = (mask == torch.finfo(torch.float32).min).all(dim=-1, keepdim=True).expand(-1, hkv * n_rep, -1, D)
        got = out.float().cpu()
        assert torch.all(got[empty] == 0)
        assert_attention_close(torch.where(empty, torch.zeros_like(got), got), torch.where(empty, torch.zeros_like(ref), ref),
                               f"cooperative prefill D={D} S={S} window={start is not None}")


@pytest.mark.parametrize("mask_dtype", [torch.bfloat16, torch.float32])
def test_cooperative_prefill_kernel_with_a_mask_tensor(device, mask_dtype):
    """The same kernel with the additive mask the reference's models pass (llama.py:292-299): ragged lengths through
    the mask alone, a mask narrower than the longest sequence's block row, one row that is masked everywhere
    (it must come out as the average of V over the mask's columns, like the reference's softmax of equal values)."""
    B, hkv, n_rep, D, S = 16, 8, 4, 128, 64
    rng = np.random.default_rng(5)
    lens = (rng.integers(S, 900, B)).tolist()
    lens[0], lens[1] = 900, S
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=91)
    q = seeded_q(34, B, hkv * n_rep, S, D)
    qd = q.to(device)
    L = max(lens)
    mask = lengths_mask_4d(lens, S, L, mask_dtype).clone()
    mask[0, :, 5, :] = torch.finfo(mask_dtype).min  # a row with nothing to read, in the sequence that fills the mask
    # most lines are plain (0 over one stretch of columns: walked without reading the mask); these are not
    mask[5, :, :, 3:17] -= 1.5                       # finite values that are not 0
    mask[6, :, :, 10] = torch.finfo(mask_dtype).min  # a masked column inside the stretch
    mask[7, :, 40:, :4] = torch.finfo(mask_dtype).min  # rows of one row group that start at different columns
    md = mask.to(device)
    if mask_dtype == torch.bfloat16:
        assert "paged_prefill_kernel<128, 2, false, true>" in _kernel_of(cache, qd, lens, md)
    out = cache.attend(qd, attention_mask=md)
    K, V = model.dense(n_rep)
    ref = sdpa_fp32(q, K[:, :, :L], V[:, :, :L], mask.float())
    assert_attention_close(out, ref, f"cooperative prefill with a {mask_dtype} mask")


@pytest.mark.parametrize("masked", [False, True])
def test_cooperative_prefill_kernel_gives_the_same_bits_every_call(device, masked):
    """Operands come out of LDS into registers that matrix instructions of the unit before were issued from, and
    the stage a unit is read from is refilled by loads that bypass the registers: every call must give the same
    bits (a barrier per unit and the waits before it are what orders the two)."""
    B, hkv, n_rep, D, S = 16, 8, 4, 128, 64
    rng = np.random.default_rng(17)
    lens = (rng.integers(S, 400, B)).tolist()
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=93)
    q = seeded_q(35, B, hkv * n_rep, S, D)
    qd = q.to(device)
    md = None
    if masked:  # values that have to be read (not a plain causal mask)
        mask = lengths_mask_4d(lens, S, max(lens), torch.bfloat16).clone()
        mask[:, :, :, 1:9] -= 0.75
        md = mask.to(device)
    assert "paged_prefill_kernel" in _kernel_of(cache, qd, lens, md)
    first = cache.attend(qd, attention_mask=md)
    differing = 0
    for _ in range(1000):
        out = cache.attend(qd, attention_mask=md)
        differing += int(not torch.equal(out.view(torch.int16), first.view(torch.int16)))
    assert differing == 0


def test_prefill_sized_launch_with_rope_rotates_queries(device):
    from oracle import rope_ref
    from pace_mi355.llm import PagedKVCache
    from pace_mi355.ops import RotaryEmbedding
    from oracle.paged_ref import RaggedCacheModel

    B, hkv, n_rep, D, S = 16, 8, 4, 128, 64
    mod = RotaryEmbedding(None, D, 256, 10000.0)
    cache = PagedKVCache(256, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, D)
    past = 0
    for step in range(2):
        k, v = seeded_kv(70 + step, B, hkv, S, D)
        q = seeded_q(80 + step, B, hkv * n_rep, S, D)
        pos = torch.arange(past, past + S).repeat(B, 1)
        rope = mod(k.to(device), pos.to(device))
        cos, sin = rope_ref.lookup(mod.cos_cache, mod.sin_cache, pos, torch.bfloat16)
        cache.update_cache(k.to(device), v.to(device), 2, rope=rope)
        model.append(rope_ref.rotate(k, cos, sin), v)
        out = cache.attend(q.to(device))
        assert_attention_close(out, model.attention(rope_ref.rotate(q, cos, sin), n_rep), f"chunk {step}")
        past += S


def test_very_long_context_single_sequence(device):
    """One sequence of 70 k tokens: many partitions per sequence, block ids beyond one wave's
    register window, the merge kernel over dozens of partials."""
    lens = [70001]
    cache, model = _build(device, 1, 2, 4, 128, lens, seed=5)
    q = seeded_q(6, 1, 8, 1, 128)
    assert_attention_close(cache.attend(q.to(device)), model.attention(q, 4), "70k decode")
    k1, v1 = seeded_kv(7, 1, 2, 3, 128)
    q3 = seeded_q(8, 1, 8, 3, 128)
    cache.update_cache(k1.to(device), v1.to(device), 2)   # fused 3-token verify on top
    model.append(k1, v1)
    assert_attention_close(cache.attend(q3.to(device)), model.attention(q3, 4), "70k verify")


@pytest.mark.parametrize("D,hkv,n_rep,lens,partition,S", [
    (128, 2, 4, [4100, 900], 64, 1),     # 65 partitions: more than one round of 64 (max, sum) pairs
    (128, 1, 8, [833], 64, 1),           # 14 partitions: a last group of fewer than eight
    (64, 2, 7, [3000], 128, 1),          # head_dim 64: half the lanes own dims
    (256, 2, 2, [2500, 64], 128, 1),     # head_dim 256: two dim pairs per lane; a sequence of one partition beside it
    (128, 2, 4, [2000, 1500], 128, 5),   # several query tokens per row group
])
def test_rows_cut_into_many_partitions(device, D, hkv, n_rep, lens, partition, S):
    """More than eight partitions per row: the merge that fetches the partials in groups, four waves per row."""
    B = len(lens)
    cache, model = _build(device, B, hkv, n_rep, D, lens, seed=sum(lens) + D, partition=partition)
    if S == 1:
        q = seeded_q(31, B, hkv * n_rep, 1, D)
        out, ref = cache.attend(q.to(device)), model.attention(q, n_rep)
    else:
        k1, v1 = seeded_kv(32, B, hkv, S, D)
        q = seeded_q(33, B, hkv * n_rep, S, D)
        cache.update_cache(k1.to(device), v1.to(device), 2)
        model.append(k1, v1)
        out, ref = cache.attend(q.to(device)), model.attention(q, n_rep)
    assert_attention_close(out, ref, f"many partitions D={D} lens={lens}")
    again = cache.attend(q.to(device)) if S == 1 else None
    if again is not None:
        assert torch.equal(out.view(torch.int16), again.view(torch.int16))


@pytest.mark.parametrize("seed", range(5))
def test_paged_attention_random_batches_masks_and_partitions(device, seed):
    """Seeded sweep: ragged lengths, query lengths on both sides of the kernel's tile limits, forced
    partition sizes, with and without an explicit mask (random bias, causal, left padding), with the
    step's tokens held back for the attention launch or appended first."""
    from pace_mi355.llm import PagedKVCache

    rng = np.random.default_rng(2000 + seed)
    for case in range(6):
        B = int(rng.integers(1, 5))
        hkv, n_rep, D = int(rng.choice([1, 2, 4])), int(rng.choice([1, 4, 8])), int(rng.choice([64, 96, 128, 128, 256]))
        S = int(rng.choice([1, 2, 5, 8, 16, 24, 70]))
        past = rng.integers(0, 400, size=B)
        uniform = rng.random() < 0.5
        if uniform:
            past[:] = past[0]
        lens = (past + S).tolist()
        Lmax = max(lens)
        tag = f"seed {seed} case {case}: B{B} hkv{hkv} rep{n_rep} D{D} S{S} lens{lens}"
        k, v = seeded_kv(seed * 100 + case, B, hkv, Lmax, D)
        q = seeded_q(seed * 100 + case + 50, B, hkv * n_rep, S, D)
        cache = PagedKVCache(Lmax + 64, num_kv_heads=hkv, n_rep=n_rep)
        cache.partition_tokens = int(rng.choice([0, 32, 128]))
        cache.fuse_append = bool(rng.random() < 0.5)
        model = RaggedCacheModel(B, hkv, D)
        if past.max() > 0:
            cache.append_ragged(k[:, :, : past.max()].to(device), v[:, :, : past.max()].to(device), past.tolist())
            model.append(k[:, :, : past.max()], v[:, :, : past.max()], past.tolist())
        kn, vn = seeded_kv(seed * 100 + case + 70, B, hkv, S, D)
        cache.update_cache(kn.to(device), vn.to(device), 2)
        model.append(kn, vn)
        kind = str(rng.choice(["none", "bias", "causal", "left-padded"]))
        if kind == "none" or not uniform:  # an explicit mask addresses columns by position: equal lengths only
            out = cache.attend(q.to(device))
            ref = model.attention(q, n_rep)
        else:
            L = lens[0]
            mdt = torch.bfloat16 if rng.random() < 0.6 else torch.float32
            m = torch.zeros(B, 1, S, L, dtype=mdt)
            if kind != "bias":
                m = causal_mask_4d(torch.ones(B, L, dtype=torch.long), S, L, mdt)
            if kind == "left-padded" and L > S + 2:
                for b in range(B):
                    m[b, :, :, : int(rng.integers(0, L - S))] = torch.finfo(mdt).min
            m = m + torch.randn(m.shape, generator=torch.Generator().manual_seed(case)).to(mdt) * (m == 0)
            out = cache.attend(q.to(device), m.to(device))
            K, V = model.dense(n_rep)
            ref = sdpa_fp32(q, K, V, m)
            tag += f" mask {kind} {mdt}"
        assert_attention_close(out, ref, tag)
        gk, gv = cache.gather(n_rep=1)
        Kd, Vd = model.dense()
        assert torch.equal(gk.cpu(), Kd) and torch.equal(gv.cpu(), Vd), tag
