"""GPU parity: paged append / gather / truncate / evict / compact / beam reorder,
bit-exact against the contiguous-semantics oracle."""
import numpy as np
import pytest
import torch

from helpers import assert_attention_close, assert_bits_equal, seeded_kv, seeded_q
from oracle.cache_ref import DynamicKVCacheRef, repeat_kv, valid_prefix
from oracle.paged_ref import RaggedCacheModel

pytestmark = pytest.mark.gpu


def _paged(max_len, **kw):
    from pace_mi355.llm import PagedKVCache

    return PagedKVCache(max_len, **kw)


@pytest.mark.parametrize("hkv,n_rep,dim", [(8, 4, 128), (2, 1, 64), (4, 8, 128), (4, 1, 256), (2, 4, 96), (2, 2, 80)])
def test_append_matches_reference_dynamic_cache(device, hkv, n_rep, dim):
    """Feed the same GQA-expanded stream to the reference's DynamicKVCache restatement
    and to the paged cache; gather(expand) must equal the reference tensors bit for bit."""
    B = 3
    ref = DynamicKVCacheRef(256)
    cache = _paged(256, num_kv_heads=hkv, n_rep=n_rep)
    for step, T in enumerate([37, 1, 1, 16, 5, 1]):
        k, v = seeded_kv(100 + step, B, hkv, T, dim)
        k_exp, v_exp = repeat_kv(k, n_rep), repeat_kv(v, n_rep)
        rk, rv = ref.update_cache(k_exp, v_exp, concat_dim=2)
        pk, pv = cache.update_cache(k_exp.to(device), v_exp.to(device), concat_dim=2)
        assert cache.seq_len == ref.seq_len
        assert_bits_equal(pk.dense(), rk, f"K after step {step}")
        assert_bits_equal(pv.dense(), rv, f"V after step {step}")
    ref.remove_cache(7)
    cache.remove_cache(7)
    rk, rv = valid_prefix(ref)
    assert_bits_equal(cache.key.dense(), rk, "K after remove_cache")
    assert_bits_equal(cache.value.dense(), rv, "V after remove_cache")
    with pytest.raises(ValueError, match="Cannot remove more tokens than available in cache."):
        cache.remove_cache(10_000)
    with pytest.raises(AssertionError, match="concat_dim should be the same"):
        cache.update_cache(k_exp.to(device), v_exp.to(device), concat_dim=1)


def test_append_from_transposed_views(device):
    """The models hand in [B,T,H,D] storage viewed as [B,H,T,D] (llama.py:125-138)."""
    B, H, T, D = 2, 4, 9, 128
    g = torch.Generator().manual_seed(7)
    base_k = torch.randn(B, T, H, D, generator=g).to(torch.bfloat16)
    base_v = torch.randn(B, T, H, D, generator=g).to(torch.bfloat16)
    cache = _paged(64)
    pk, pv = cache.update_cache(base_k.to(device).transpose(1, 2), base_v.to(device).transpose(1, 2), concat_dim=2)
    assert_bits_equal(pk.dense(), base_k.transpose(1, 2).contiguous(), "K")
    assert_bits_equal(pv.dense(), base_v.transpose(1, 2).contiguous(), "V")


def test_ragged_append_truncate_evict_compact(device):
    B, H, D = 5, 2, 128
    rng = np.random.default_rng(11)
    cache = _paged(400, num_blocks=160)
    model = RaggedCacheModel(B, H, D)
    for step in range(6):
        T = int(rng.integers(1, 40))
        counts = rng.integers(0, T + 1, size=B)
        k, v = seeded_kv(200 + step, B, H, T, D)
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
    assert cache.lens.tolist() == model.seq_lens()
    check("after evict")
    moved = cache.compact()
    live = cache.state.live_block_count()
    used = np.concatenate([cache.state.table[b, : cache.state.n_blocks[b]] for b in range(B)])
    assert sorted(used.tolist()) == list(range(live)), "live blocks must occupy ids 0..n_live-1"
    assert moved <= live
    check("after compact")
    # appending after compaction reuses freed ids correctly
    k, v = seeded_kv(300, B, H, 20, D)
    cache.append_ragged(k.to(device), v.to(device), [20] * B)
    model.append(k, v)
    check("after post-compaction append")


@pytest.mark.parametrize("hkv,n_rep,dim", [(2, 1, 128), (8, 4, 128), (2, 2, 64), (1, 3, 256), (2, 1, 80)])
def test_packed_gather_and_gather_without_zero_fill(device, hkv, n_rep, dim):
    """The two gather forms that write no padding: packed [sum len][H][D] with cu_seqlens, and the
    dense layout with the rows past each length left alone.  Both bit-exact on every row a sequence has."""
    B = 6
    rng = np.random.default_rng(5)
    lens = [0, 1, 16, 17, 333, 40]
    cache = _paged(400, num_kv_heads=hkv, n_rep=n_rep)
    model = RaggedCacheModel(B, hkv, dim)
    k, v = seeded_kv(77, B, hkv, max(lens), dim)
    cache.append_ragged(k.to(device), v.to(device), lens)
    model.append(k, v, lens)
    cache.truncate([0, 0, 3, 0, 13, 0])
    model.truncate([0, 0, 3, 0, 13, 0])
    lens = model.seq_lens()
    for rep in (1, n_rep):
        K, V = model.dense(rep)
        pk, pv, cu = cache.gather_packed(n_rep=rep)
        assert cu.cpu().tolist() == np.concatenate([[0], np.cumsum(lens)]).tolist()
        assert tuple(pk.shape) == (sum(lens), hkv * rep, dim)
        want_k = torch.cat([K[b, :, :n].transpose(0, 1) for b, n in enumerate(lens)], dim=0)
        want_v = torch.cat([V[b, :, :n].transpose(0, 1) for b, n in enumerate(lens)], dim=0)
        assert_bits_equal(pk, want_k, f"packed K n_rep={rep}")
        assert_bits_equal(pv, want_v, f"packed V n_rep={rep}")
        gk, gv = cache.gather(n_rep=rep, zero_fill=False)
        for b, n in enumerate(lens):
            assert_bits_equal(gk[b, :, :n], K[b, :, :n], f"K rows of sequence {b}")
            assert_bits_equal(gv[b, :, :n], V[b, :, :n], f"V rows of sequence {b}")


def test_gather_without_zero_fill_leaves_padding_untouched(device):
    import ctypes

    from pace_mi355 import _native as nat

    B, H, D, L = 2, 2, 128, 40
    cache = _paged(64)
    k, v = seeded_kv(3, B, H, 30, D)
    cache.append_ragged(k.to(device), v.to(device), [30, 5])
    st = cache.state
    table, (lens_dev, bias) = st.device_table(), st.device_lens(cache.lens)
    outs = [torch.full((B, H, L, D), 3.0, dtype=torch.bfloat16, device=device) for _ in range(2)]
    nat.check(nat.load().pace_kv_gather(ctypes.byref(cache._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias, B, 1,
                                        outs[0].data_ptr(), outs[1].data_ptr(), outs[0].stride(0), outs[0].stride(1), L, 0,
                                        nat.current_stream_ptr()))
    torch.cuda.synchronize()
    for o, src in zip(outs, (k, v)):
        assert_bits_equal(o[0, :, :30], src[0, :, :30], "rows of sequence 0")
        assert_bits_equal(o[1, :, :5], src[1, :, :5], "rows of sequence 1")
        assert bool((o[0, :, 30:] == 3.0).all()) and bool((o[1, :, 5:] == 3.0).all()), "padding rows were written"


@pytest.mark.parametrize("out_len", [40, 12])
def test_gather_over_the_blocks_that_exist_writes_only_rows_that_exist(device, out_len):
    """pace_kv_gather_live: the dense layout written from the grid of the packed form.  Rows below
    min(len, out_len) bit-exact; padding rows, rows of an empty sequence and the memory behind the
    outputs untouched -- also when out_len cuts a sequence short."""
    import ctypes

    from pace_mi355 import _native as nat

    B, H, D, rep = 4, 2, 128, 2
    lens = [30, 0, 5, 17]
    cache = _paged(64)
    k, v = seeded_kv(3, B, H, max(lens), D)
    cache.append_ragged(k.to(device), v.to(device), lens)
    st = cache.state
    table, (lens_dev, bias) = st.device_table(), st.device_lens(cache.lens)
    cu = torch.tensor(np.concatenate([[0], np.cumsum(lens)]), dtype=torch.int32, device=device)
    guard = 3 * D
    flat = [torch.full((B * H * rep * out_len * D + guard,), 3.0, dtype=torch.bfloat16, device=device) for _ in range(2)]
    outs = [f[: B * H * rep * out_len * D].view(B, H * rep, out_len, D) for f in flat]
    nat.check(nat.load().pace_kv_gather_live(ctypes.byref(cache._desc), table.data_ptr(), table.stride(0), lens_dev.data_ptr(), bias,
                                             cu.data_ptr(), B, rep, outs[0].data_ptr(), outs[1].data_ptr(), outs[0].stride(0),
                                             outs[0].stride(1), out_len, sum(lens), nat.current_stream_ptr()))
    torch.cuda.synchronize()
    for f, o, src in zip(flat, outs, (k, v)):
        want = src.repeat_interleave(rep, dim=1)
        for b, n in enumerate(lens):
            m = min(n, out_len)
            assert_bits_equal(o[b, :, :m], want[b, :, :m], f"rows of sequence {b}")
            assert bool((o[b, :, m:] == 3.0).all()), f"rows past the end of sequence {b} were written"
        assert bool((f[-guard:] == 3.0).all()), "memory behind the outputs was written"


def test_beam_reorder(device):
    B, H, D = 4, 2, 64
    cache = _paged(128, num_blocks=80)
    model = RaggedCacheModel(B, H, D)
    k, v = seeded_kv(5, B, H, 45, D)
    cache.update_cache(k.to(device), v.to(device), 2)
    model.append(k, v)
    idx = [2, 2, 0, 3]
    cache.update_cache_with_beam_indices(torch.tensor(idx))
    model.reorder(idx)
    K, V = model.dense()
    gk, gv = cache.gather()
    assert_bits_equal(gk, K, "K after beam reorder")
    assert_bits_equal(gv, V, "V after beam reorder")


def test_beam_search_steps_copy_on_write(device):
    """Several reorder / append rounds as beam search issues them (pace/llm/generator.py:606-610):
    contents equal the reference's index_select semantics bit for bit, while only the block each
    beam writes into is ever copied."""
    B, H, D = 4, 2, 128
    cache = _paged(256, num_blocks=64)
    model = RaggedCacheModel(B, H, D)
    k, v = seeded_kv(50, B, H, 37, D)
    cache.update_cache(k.to(device), v.to(device), 2)
    model.append(k, v)
    q = seeded_q(51, B, H, 1, D)

    def check(what):
        K, V = model.dense()
        gk, gv = cache.gather()
        assert_bits_equal(gk, K, "K " + what)
        assert_bits_equal(gv, V, "V " + what)

    plans = [[0, 0, 2, 1], [3, 3, 3, 0], [0, 1, 2, 3], [1, 0, 0, 0], [2, 2, 1, 1], [0, 0, 0, 0]]
    for step, idx in enumerate(plans * 3):
        cache.update_cache_with_beam_indices(torch.tensor(idx))
        model.reorder(idx)
        check(f"after reorder {step}")
        k, v = seeded_kv(60 + step, B, H, 1, D)
        cache.update_cache(k.to(device), v.to(device), 2)
        model.append(k, v)
        out = cache.attend(q.to(device))
        assert_attention_close(out, model.attention(q, 1), f"decode after reorder {step}")
        check(f"after append {step}")
    # 18 steps x 4 beams: at most one block per beam and step, none when a beam kept its own tail
    assert 0 < cache.cow_blocks_copied <= 18 * 4
    used = cache.state.live_block_count()
    assert used <= 4 * 4 + 4, f"{used} blocks in use: forks must share their common prefix"
    # rollback and eviction on top of shared blocks
    cache.truncate([3, 0, 20, 1])
    model.truncate([3, 0, 20, 1])
    k, v = seeded_kv(90, B, H, 5, D)
    cache.update_cache(k.to(device), v.to(device), 2)
    model.append(k, v)
    check("after rollback + append")
    cache.evict_blocks(1, [0])
    model.evict_blocks(1, [0], 16)
    cache.compact()
    check("after evict + compact")
    k, v = seeded_kv(91, B, H, 2, D)
    cache.update_cache(k.to(device), v.to(device), 2)
    model.append(k, v)
    check("after the last append")


def test_manager_layers_share_block_table(device):
    from pace_mi355.llm import KVCacheManager, KVCacheType

    class Cfg:
        num_hidden_layers = 2
        num_attention_heads = 8
        num_key_value_heads = 2

    mgr = KVCacheManager(Cfg(), 96, KVCacheType.PAGED)
    refs = [DynamicKVCacheRef(96) for _ in range(2)]
    for step, T in enumerate([30, 1, 1]):
        for layer in range(2):
            k, v = seeded_kv(400 + 10 * step + layer, 2, 2, T, 128)
            ke, ve = repeat_kv(k, 4), repeat_kv(v, 4)
            refs[layer].update_cache(ke, ve, 2)
            mgr[layer].update_cache(ke.to(device), ve.to(device), 2)
        assert len(mgr) == refs[0].seq_len
    mgr.remove_cache(3)
    for layer in range(2):
        refs[layer].remove_cache(3)
        rk, rv = valid_prefix(refs[layer])
        assert_bits_equal(mgr[layer].key.dense(), rk, f"layer {layer} K")
        assert_bits_equal(mgr[layer].value.dense(), rv, f"layer {layer} V")
    assert mgr[0].state is mgr[1].state


@pytest.mark.parametrize("seed", [0, 1])
def test_random_histories_with_real_data(device, seed):
    """A random run of uniform (fused) and ragged appends, rollbacks, evictions, compactions and beam
    re-orderings: after every step the dense view equals the oracle's cache bit for bit, and decode
    attention over it matches the oracle."""
    B, H, n_rep, D = 4, 2, 4, 128
    rng = np.random.default_rng(100 + seed)
    cache = _paged(640, num_kv_heads=H, n_rep=n_rep, num_blocks=220)
    model = RaggedCacheModel(B, H, D)
    k, v = seeded_kv(400 + seed, B, H, 24, D)
    cache.append_ragged(k.to(device), v.to(device), [24, 7, 16, 1])
    model.append(k, v, [24, 7, 16, 1])
    for step in range(40):
        op = rng.choice(["uniform", "uniform", "ragged", "truncate", "evict", "compact", "reorder"])
        if max(model.seq_lens()) > 560 and op in ("uniform", "ragged"):
            op = "truncate"
        if op == "uniform":  # what a decode / verify step does: held back and stored by the attention launch
            T = int(rng.choice([1, 1, 4, 9, 33]))
            k, v = seeded_kv(1000 * seed + 2 * step, B, H, T, D)
            cache.update_cache(k.to(device), v.to(device), 2)
            model.append(k, v)
            q = seeded_q(1000 * seed + 2 * step + 1, B, H * n_rep, T, D)
            assert_attention_close(cache.attend(q.to(device)), model.attention(q, n_rep), f"step {step} attention after {T}-token append")
        elif op == "ragged":
            T = int(rng.integers(1, 30))
            counts = rng.integers(0, T + 1, size=B)
            k, v = seeded_kv(1000 * seed + 2 * step, B, H, T, D)
            cache.append_ragged(k.to(device), v.to(device), counts)
            model.append(k, v, counts)
        elif op == "truncate":
            rem = [int(rng.integers(0, min(40, n + 1))) for n in model.seq_lens()]
            cache.truncate(rem)
            model.truncate(rem)
        elif op == "evict":
            b = int(rng.integers(0, B))
            nb = (model.seq_lens()[b] + 15) // 16
            if nb == 0:
                continue
            drop = sorted(set(rng.integers(0, nb, size=int(rng.integers(1, 4))).tolist()))
            cache.evict_blocks(b, drop)
            model.evict_blocks(b, drop, 16)
        elif op == "compact":
            cache.compact()
        else:
            idx = rng.integers(0, B, size=B).tolist()
            cache.reorder(idx)
            model.reorder(idx)
        assert cache.lens.tolist() == model.seq_lens(), f"step {step} ({op})"
        K, V = model.dense()
        gk, gv = cache.gather(n_rep=1)
        assert_bits_equal(gk, K, f"K after step {step} ({op})")
        assert_bits_equal(gv, V, f"V after step {step} ({op})")
    # Copy-on-write by construction, whatever the history above happened to do: every sequence is brought to a
    # partly filled last block, sequences 1 and 3 become copies of 0 and 2, and a uniform append follows.  The first
    # writer of each shared tail block must get a private copy of it (one block per pair), the second then owns the
    # original alone; the dense view and the attention over it must still match the oracle.
    counts = [(5 - n) % 16 for n in model.seq_lens()]
    k, v = seeded_kv(9000 + seed, B, H, 16, D)
    cache.append_ragged(k.to(device), v.to(device), counts)
    model.append(k, v, counts)
    cache.reorder([0, 0, 2, 2])
    model.reorder([0, 0, 2, 2])
    copied_before = cache.cow_blocks_copied
    k, v = seeded_kv(9100 + seed, B, H, 1, D)
    cache.update_cache(k.to(device), v.to(device), 2)
    model.append(k, v)
    q = seeded_q(9200 + seed, B, H * n_rep, 1, D)
    assert_attention_close(cache.attend(q.to(device)), model.attention(q, n_rep), "attention after the forced copy-on-write")
    assert cache.cow_blocks_copied == copied_before + 2
    K, V = model.dense()
    gk, gv = cache.gather(n_rep=1)
    assert_bits_equal(gk, K, "K after the forced copy-on-write")
    assert_bits_equal(gv, V, "V after the forced copy-on-write")
