"""CPU tests of the host side: operator registry, enums, cache-manager interface,
contiguous caches vs the oracle, block allocator and eviction / compaction plans."""
import re

import ctypes

import numpy as np
import pytest
import torch

from oracle.cache_ref import BMCKVCacheRef, DynamicKVCacheRef, valid_prefix
from pace_mi355.llm import (
    BMCKVCache,
    DynamicKVCache,
    KVCacheManager,
    KVCacheType,
    LLMBackendType,
    LLMOperatorType,
    PagedKVCache,
    get_kv_cache_class,
)
from pace_mi355.llm.paged import BlockAllocator, PagedState
from pace_mi355.ops import BackendType, DataType, FusedOperatorType, MultiHeadAttention, OperatorType, backend_registry
from pace_mi355.ops import enum as ops_enum
from pace_mi355.ops.base import BackendBase
from pace_mi355.ops.registry import BackendRegistry


# ---- registry (semantics of the reference's tests/python_ops/test_registry.py) ----
class _A:  # dummy implementations
    pass


class _B:
    pass


@pytest.fixture()
def registry():
    saved = list(ops_enum.FALLBACK_BACKEND)
    yield BackendRegistry()
    ops_enum.FALLBACK_BACKEND[:] = saved


def test_register_and_get_every_combination(registry):
    for op in OperatorType:
        for be in BackendType:
            cls = type("Impl", (), {})
            registry.register(op, be, list(DataType))(cls)
            for dt in DataType:
                assert registry.get(op, be, dt) is cls


def test_unregistered_operator_gives_none(registry):
    assert registry.get(OperatorType.MHA, BackendType.JIT, DataType.BFLOAT16) is None
    assert registry.get_available_backends(OperatorType.MHA) == []


def test_fallback_order(registry):
    op, dt = OperatorType.MHA, DataType.BFLOAT16
    registry.register(op, BackendType.NATIVE, [dt])(_A)
    registry.register(op, BackendType.JIT, [dt])(_B)
    ops_enum.FALLBACK_BACKEND[:] = [BackendType.JIT, BackendType.NATIVE]
    assert registry.get(op, BackendType.TPP, dt) is _B
    ops_enum.FALLBACK_BACKEND[:] = [BackendType.NATIVE, BackendType.JIT]
    assert registry.get(op, BackendType.TPP, dt) is _A
    assert registry.get(op, BackendType.JIT, dt) is _B  # exact match wins over fallback


def test_fused_operators_never_fall_back(registry):
    registry.register(FusedOperatorType.FUSEDLINEARGELU, BackendType.TPP, [DataType.BFLOAT16])(_A)
    assert registry.get(FusedOperatorType.FUSEDLINEARGELU, BackendType.TPP, DataType.BFLOAT16) is _A
    assert registry.get(FusedOperatorType.FUSEDLINEARGELU, BackendType.JIT, DataType.BFLOAT16) is None
    assert registry.get(FusedOperatorType.FUSEDLINEARGELU, BackendType.TPP, DataType.FLOAT32) is None


def test_duplicate_and_missing_assert(registry):
    registry.register(OperatorType.LINEAR, BackendType.JIT, [DataType.BFLOAT16])(_A)
    with pytest.raises(AssertionError, match="Duplicate registration"):
        registry.register(OperatorType.LINEAR, BackendType.JIT, [DataType.BFLOAT16])
    ops_enum.FALLBACK_BACKEND[:] = [BackendType.TPP]
    with pytest.raises(AssertionError, match="No backend found for linear with jit, float32"):
        registry.get(OperatorType.LINEAR, BackendType.JIT, DataType.FLOAT32)


def test_registry_repr(registry):
    registry.register(OperatorType.LINEAR, BackendType.NATIVE, [DataType.BFLOAT16])(_A)
    text = repr(registry)
    for needle in ("OperatorType.LINEAR", "BackendType.NATIVE", "DataType.BFLOAT16", "_A"):
        assert needle in text


def test_enums_are_lowercase_strings():
    assert OperatorType.MHA == "mha" and f"{BackendType.HIP}" == "hip" and str(DataType.BFLOAT16) == "bfloat16"
    assert [b.name for b in BackendType][:4] == ["NATIVE", "JIT", "TPP", "IMBPS"]
    assert DataType.from_torch(torch.bfloat16) is DataType.BFLOAT16 and DataType.FLOAT32.to_torch_dtype() is torch.float32
    with pytest.raises(ValueError, match="Unsupported dtype"):
        DataType.from_torch(torch.int8)
    assert LLMBackendType is BackendType and LLMOperatorType.Attention == "attention"


def test_mha_resolves_to_hip_backend_whatever_backend_is_asked():
    from pace_mi355.ops.backends.hip import HIPAttention

    assert set(backend_registry.get_available_backends(OperatorType.MHA)) == {
        (BackendType.HIP, DataType.FLOAT32), (BackendType.HIP, DataType.BFLOAT16)}
    for be in BackendType:
        mha = MultiHeadAttention(backend_impl=be, dtype=torch.bfloat16)
        assert isinstance(mha.backend, HIPAttention) and isinstance(mha.backend, BackendBase)
        assert mha.operator_type is OperatorType.MHA
        assert "HIPAttention" in repr(mha)


# ---- cache-manager interface ----
class _Cfg:
    num_hidden_layers = 2


def test_cache_type_enum_and_class_lookup():
    assert KVCacheType("dynamic") is KVCacheType.DYNAMIC and KVCacheType("bmc") is KVCacheType.BMC
    assert KVCacheType.get_kv_cache_type("paged") is KVCacheType.PAGED
    assert get_kv_cache_class("dynamic") is DynamicKVCache and get_kv_cache_class(KVCacheType.BMC) is BMCKVCache
    assert get_kv_cache_class("paged") is PagedKVCache
    with pytest.raises(ValueError):
        KVCacheType("nope")


def test_manager_interface_matches_reference_expectations():
    mgr = KVCacheManager(_Cfg(), 128, KVCacheType.DYNAMIC)
    assert len(mgr.cache_objects) == 2 and isinstance(mgr[0], DynamicKVCache) and len(mgr) == 0
    assert mgr.update_mask(torch.ones(2, 10), 10).shape == (2, 10)
    bmc = BMCKVCache(128)
    k, v = bmc.update_cache(torch.rand(2, 10, 64), torch.rand(2, 10, 64), concat_dim=1)
    assert k.shape[1] == 11 and v.shape[1] == 11
    assert bmc.update_mask(torch.ones(2, 10), 10).shape == (2, 11)
    dyn = DynamicKVCache(128)
    k, v = dyn.update_cache(torch.rand(2, 10, 64), torch.rand(2, 10, 64), concat_dim=1)
    assert k.shape[1] == 10
    paged = KVCacheManager(_Cfg(), 128, "paged")
    assert isinstance(paged[1], PagedKVCache) and len(paged) == 0
    paged.remove_cache(3)  # empty caches ignore removal, like the reference


@pytest.mark.parametrize("prod,ref", [(DynamicKVCache, DynamicKVCacheRef), (BMCKVCache, BMCKVCacheRef)])
def test_contiguous_caches_track_the_oracle(prod, ref):
    g = torch.Generator().manual_seed(3)
    a, b = prod(200), ref(200)
    for T in (13, 1, 1, 30, 2):
        k, v = torch.randn(2, 3, T, 4, generator=g), torch.randn(2, 3, T, 4, generator=g)
        ka, va = a.update_cache(k, v, 2)
        kb, vb = b.update_cache(k, v, 2)
        assert torch.equal(ka, kb) and torch.equal(va, vb) and a.seq_len == b.seq_len
    a.remove_cache(5), b.remove_cache(5)
    assert torch.equal(a.key.narrow(2, 0, a.seq_len), valid_prefix(b)[0])
    k = torch.randn(2, 3, 1, 4, generator=g)
    assert torch.equal(a.update_cache(k, k, 2)[0], b.update_cache(k, k, 2)[0])
    m = torch.zeros(2, 1, 1, a.seq_len, dtype=torch.bfloat16)
    assert torch.equal(a.update_mask(m, a.seq_len), b.update_mask(m, b.seq_len))
    with pytest.raises(ValueError, match="Cannot remove more tokens than available in cache."):
        a.remove_cache(10_000)
    with pytest.raises(AssertionError, match="concat_dim should be the same for all updates"):
        a.update_cache(k, k, 1)
    idx = torch.tensor([1, 1])
    a.update_cache_with_beam_indices(idx), b.update_cache_with_beam_indices(idx)
    assert torch.equal(a.key, b.key)


def test_paged_cache_refuses_cpu_tensors():
    with pytest.raises(RuntimeError, match="GPU memory"):
        PagedKVCache(64).update_cache(torch.zeros(1, 1, 1, 128, dtype=torch.bfloat16), torch.zeros(1, 1, 1, 128, dtype=torch.bfloat16), 2)


# ---- allocator and plans ----
def test_allocator_lifo_and_errors():
    al = BlockAllocator(6)
    assert al.allocate(3) == [0, 1, 2] and al.num_free == 3
    al.free([1])
    assert al.allocate(1) == [1]
    with pytest.raises(ValueError, match="freed twice"):
        al.free([5])
    with pytest.raises(MemoryError, match="exhausted"):
        al.allocate(4)
    al.take([4])
    assert sorted(al.free_ids().tolist()) == [3, 5]
    with pytest.raises(ValueError, match="not free"):
        al.take([0])


def _state(batch=3, max_len=160, blocks=40):
    return PagedState(batch, max_len, blocks, torch.device("cpu"))


def test_capacity_release_and_slots():
    st = _state()
    lens = np.array([33, 16, 0])
    st.ensure_capacity(lens)
    assert st.n_blocks.tolist() == [3, 1, 0] and st.allocator.num_free == 36
    assert st.min_capacity == 0  # the empty sequence owns no block yet
    st2 = _state()
    st2.ensure_capacity(np.array([33, 16, 5]))
    assert st2.min_capacity == 16  # what every sequence can hold without a new block
    s = st.slots(np.array([30, 0, 0]), np.array([3, 2, 0]), 4)
    assert s[0].tolist() == [st.table[0, 1] * 16 + 14, st.table[0, 1] * 16 + 15, st.table[0, 2] * 16, -1]
    assert s[1].tolist()[:2] == [st.table[1, 0] * 16, st.table[1, 0] * 16 + 1] and (s[2] == -1).all()
    assert st.release_beyond(np.array([16, 16, 0])) == 2 and st.n_blocks.tolist() == [1, 1, 0]
    with pytest.raises(MemoryError, match="pool exhausted"):
        st.ensure_capacity(np.array([16, 16, 2000]))


@pytest.mark.parametrize("seed", range(4))
def test_capacity_changes_over_the_batch_match_one_sequence_at_a_time(seed):
    """ensure_capacity / release_beyond handle the whole batch in one allocation / one release: the block ids every
    sequence ends up with, the reference counts and the order of the free list are those of taking the sequences
    one by one (one allocate() or free() per sequence, in batch order), forks included."""
    rng = np.random.default_rng(seed)
    B = 7
    st = PagedState(B, 64, 400, torch.device("cpu"))
    ref = PagedState(B, 64, 400, torch.device("cpu"))

    def grow_one_by_one(state, lens):
        need = (lens + 15) // 16
        state._grow_table(int(need.max(initial=0)))
        for b in range(B):
            have, want = int(state.n_blocks[b]), int(need[b])
            if want > have:
                state.table[b, have:want] = state.allocator.allocate(want - have)
                state.n_blocks[b] = want

    def shrink_one_by_one(state, lens):
        need = (lens + 15) // 16
        for b in range(B):
            have, want = int(state.n_blocks[b]), int(need[b])
            if want < have:
                state.allocator.free(state.table[b, want:have].tolist())
                state.table[b, want:have] = 0
                state.n_blocks[b] = want

    lens = np.zeros(B, dtype=np.int64)
    for step in range(60):
        kind = rng.integers(0, 4)
        if kind <= 1:  # some sequences grow
            lens = lens + rng.integers(0, 90, size=B) * (rng.random(B) < 0.7)
            st.ensure_capacity(lens)
            grow_one_by_one(ref, lens)
        elif kind == 2:  # some shrink (rollback, or a sequence that ends)
            lens = (lens * rng.choice([0.0, 0.5, 1.0], size=B)).astype(np.int64)
            st.release_beyond(lens)
            shrink_one_by_one(ref, lens)
        else:  # beam step: every row continues some source row (blocks shared until written)
            src = rng.integers(0, B, size=B).tolist()
            st.fork(src)
            ref.fork(src)
            lens = lens[src]
        n = st.allocator.num_free
        assert n == ref.allocator.num_free
        assert st.allocator._stack[:n].tolist() == ref.allocator._stack[:n].tolist()
        assert st.allocator.refs.tolist() == ref.allocator.refs.tolist()
        assert st.n_blocks.tolist() == ref.n_blocks.tolist()
        for b in range(B):
            assert st.table[b, : st.n_blocks[b]].tolist() == ref.table[b, : ref.n_blocks[b]].tolist()


def test_table_grows_on_demand():
    st = PagedState(1, 16, 300, torch.device("cpu"))
    st.ensure_capacity(np.array([16 * 200]))
    assert st.n_blocks[0] == 200 and st.table.shape[1] >= 200
    assert len(set(st.table[0, :200].tolist())) == 200


def test_evict_and_compaction_plan_properties():
    rng = np.random.default_rng(5)
    st = _state(batch=4, max_len=400, blocks=120)
    lens = np.array([400, 130, 16, 77])
    st.ensure_capacity(lens)
    before = {b: st.table[b, : st.n_blocks[b]].copy() for b in range(4)}
    new_lens = st.evict(0, [1, 5, 24], lens)  # block 24 is the last (full) block of 400 tokens
    assert new_lens[0] == 400 - 48 and st.n_blocks[0] == 22
    assert st.table[0, :22].tolist() == [x for j, x in enumerate(before[0].tolist()) if j not in (1, 5, 24)]
    new_lens = st.evict(1, [8], new_lens)  # partial last block holds 2 tokens
    assert new_lens[1] == 128
    with pytest.raises(IndexError):
        st.evict(2, [3], new_lens)
    for b in range(4):  # scatter a few more holes
        n = int(st.n_blocks[b])
        if n > 2:
            new_lens = st.evict(b, sorted(rng.choice(n - 1, size=n // 3, replace=False).tolist()), new_lens)
    moves = st.plan_compaction()
    live = st.live_block_count()
    assert not (set(moves[:, 0].tolist()) & set(moves[:, 1].tolist()))
    assert (moves[:, 0] >= live).all() and (moves[:, 1] < live).all()
    logical = {b: st.table[b, : st.n_blocks[b]].copy() for b in range(4)}
    st.apply_moves(moves)
    used = np.concatenate([st.table[b, : st.n_blocks[b]] for b in range(4)])
    assert sorted(used.tolist()) == list(range(live))
    remap = dict(zip(moves[:, 0].tolist(), moves[:, 1].tolist()))
    for b in range(4):
        assert st.table[b, : st.n_blocks[b]].tolist() == [remap.get(x, x) for x in logical[b].tolist()]
    assert sorted(st.allocator.free_ids().tolist()) == list(range(live, 120))
    assert len(st.plan_compaction()) == 0  # idempotent


def test_fork_shares_blocks_and_copy_on_write_touches_only_shared_tails():
    """Beam reorder as table surgery (the reference copies the whole cache, pace/llm/cache.py:161-167)."""
    st = _state(batch=4, max_len=160, blocks=40)
    lens = np.array([40, 40, 40, 40])  # 3 blocks each, the last holds 8 tokens
    st.ensure_capacity(lens)
    rows = {b: st.table[b, :3].tolist() for b in range(4)}
    st.fork([2, 2, 0, 2])
    assert [st.table[i, :3].tolist() for i in range(4)] == [rows[2], rows[2], rows[0], rows[2]]
    assert st.allocator.refs[rows[2]].tolist() == [3, 3, 3] and st.allocator.refs[rows[0]].tolist() == [1, 1, 1]
    assert st.allocator.num_free == 40 - 6 and st.live_block_count() == 6  # rows 1 and 3 were dropped
    assert st.has_shared and st.tails_dirty
    pairs = st.unshare_tails(lens)
    # the three owners of rows[2]'s tail: two get a private copy, the last one keeps the original
    assert len(pairs) == 2 and set(pairs[:, 0].tolist()) == {rows[2][2]}
    assert st.allocator.refs[rows[2][2]] == 1 and not st.tails_dirty and st.has_shared
    tails = [int(st.table[i, 2]) for i in range(4)]
    assert len(set(tails)) == 4
    assert len(st.unshare_tails(lens)) == 0
    # full blocks stay shared; a sequence that ends on a block boundary needs no copy at all
    st2 = _state(batch=2, max_len=160, blocks=40)
    st2.ensure_capacity(np.array([32, 32]))
    st2.fork([1, 1])
    assert len(st2.unshare_tails(np.array([32, 32]))) == 0
    # rollback into a shared full block makes it a tail again
    st2.release_beyond(np.array([20, 20]))
    st2.lengths_shrank()
    assert st2.tails_dirty
    assert len(st2.unshare_tails(np.array([20, 20]))) == 1
    # dropping every owner frees the block exactly once
    st2.release_beyond(np.array([0, 0]))
    assert st2.allocator.num_free == 40 and not (st2.allocator.refs > 0).any()
    with pytest.raises(IndexError):
        st2.fork([0, 5])


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_compaction_plan_from_free_flags_and_tracked_apply_agree_with_the_table_walk(seed):
    """The planner that reads the allocator's free flags gives the moves of the planner that walks the table, and the
    apply that moves the bookkeeping along leaves what a recount leaves: the same table, owners per block, free
    flags, and a free list that hands out the lowest ids first.  Forked sequences (blocks with several owners)
    included; a move that does not take a used block to a free one is refused and nothing changes."""
    from pace_mi355 import _native as nat

    lib = nat.load()
    rng = np.random.default_rng(seed)
    B, N = 5, 157
    st = _state(batch=B, max_len=16 * 40, blocks=N)
    lens = rng.integers(1, 16 * 30, B)
    st.ensure_capacity(lens)
    for b in range(B):
        n = int(st.n_blocks[b])
        if n > 2:
            lens = st.evict(b, sorted(rng.choice(n, size=n // 3, replace=False).tolist()), lens)
    st.fork([0, 0, 2, 3, 3])  # shared blocks: owners per block above one
    lens = lens[[0, 0, 2, 3, 3]]
    alloc = st.allocator
    # the two planners
    by_table = np.empty((N, 2), np.int32)
    n1 = lib.pace_kv_plan_compaction(st.table.ctypes.data, st.table.shape[1], st.n_blocks.ctypes.data, B, N, by_table.ctypes.data, N, 0, None)
    by_flags = st.plan_compaction()
    assert n1 == len(by_flags) > 0 and np.array_equal(by_table[:n1], by_flags)
    # reference result: the recounting apply on copies
    table0, refs0 = st.table.copy(), alloc.refs.copy()
    want_table, want_refs = st.table.copy(), np.empty(N, np.int32)
    nat.check(lib.pace_kv_apply_moves(want_table.ctypes.data, want_table.shape[1], st.n_blocks.ctypes.data, B, N, by_flags.ctypes.data, n1,
                                      want_refs.ctypes.data))
    # a bad move first: destination in use -> refused, nothing touched
    bad = by_flags.copy()
    bad[-1, 1] = by_flags[0, 0]
    flags0, stack0, nfree0 = alloc._is_free.copy(), alloc._stack.copy(), alloc.num_free
    with pytest.raises(Exception, match="does not take a live block to a free one"):
        st.apply_moves(bad)
    assert np.array_equal(st.table, table0) and np.array_equal(alloc.refs, refs0) and np.array_equal(alloc._is_free, flags0)
    assert np.array_equal(alloc._stack, stack0) and alloc.num_free == nfree0
    st.apply_moves(by_flags)
    assert np.array_equal(st.table, want_table) and np.array_equal(alloc.refs, want_refs)
    assert np.array_equal(alloc._is_free, want_refs == 0) and alloc.num_free == int((want_refs == 0).sum())
    live = st.live_block_count()
    assert sorted(alloc.free_ids().tolist()) == list(range(live, N))
    assert alloc.allocate(3) == [live, live + 1, live + 2], "the lowest free ids are handed out first"
    assert len(st.plan_compaction()) == 0


def test_compaction_moves_a_shared_block_once():
    st = _state(batch=3, max_len=160, blocks=30)
    st.ensure_capacity(np.array([48, 48, 48]))
    st.fork([0, 0, 2])            # blocks of old row 1 are freed: holes at ids 3..5
    moves = st.plan_compaction()
    assert st.live_block_count() == 6 and len(moves) == 3
    shared_before = st.table[0, :3].tolist()
    st.apply_moves(moves)
    assert st.table[0, :3].tolist() == st.table[1, :3].tolist()
    remap = dict(zip(moves[:, 0].tolist(), moves[:, 1].tolist()))
    assert st.table[0, :3].tolist() == [remap.get(x, x) for x in shared_before]
    assert st.allocator.refs[st.table[0, :3]].tolist() == [2, 2, 2]
    assert sorted(st.allocator.free_ids().tolist()) == list(range(6, 30))


# ---- attention launch planning (the library's host-side planner; no GPU involved) ----
def _planned(st, lens, hq=32, hkv=8, dim=128, q_len=1, masked=False, partition=0):
    lens = np.asarray(lens, dtype=np.int64)
    st.ensure_capacity(lens)
    items, parts, n, max_parts, ws = st.plan_attention(lens, hq, hkv, dim, q_len, masked, partition)
    it = items.numpy().reshape(-1, 16)
    assert it.shape[0] == n
    return it, parts.numpy(), max_parts, ws


def _check_cover(it, parts, lens, table):
    """Every sequence is cut into its partitions exactly once: contiguous ranges of whole 32-token units from
    token 0, the last one open ended; the unit entries name the table's blocks."""
    lens = np.asarray(lens)
    assert sorted(map(tuple, it[:, :2].tolist())) == sorted((b, p) for b in range(len(lens)) for p in range(parts[b]))
    for b in range(len(lens)):
        rows = it[it[:, 0] == b]
        rows = rows[np.argsort(rows[:, 1])]
        assert (rows[:, 2] == parts[b]).all()
        assert rows[0, 3] == 0 and (rows[:, 3] % 32 == 0).all()
        assert (rows[:-1, 4] == rows[1:, 3]).all() and rows[-1, 4] == -1
        assert (rows[:, 3] < max(lens[b], 1)).all(), "no partition may be empty"
        for r in rows:
            end = lens[b] if r[4] < 0 else r[4]
            whole = min(4, max(0, (end - r[3]) // 32))
            assert r[5] == whole
            for u in range(4):
                j = r[3] // 16 + 2 * u
                want = table[b, j:j + 2].tolist() if u < whole else [0, 0]
                assert r[8 + 2 * u: 10 + 2 * u].tolist() == want


def test_plan_attention_uniform_batch_is_cut_evenly_in_table_order():
    st = _state(batch=4, max_len=8192, blocks=4 * 520)
    lens = np.full(4, 4097)
    it, parts, max_parts, ws = _planned(st, lens)
    _check_cover(it, parts, lens, st.table)
    assert (parts == parts[0]).all() and max_parts == parts[0] > 1          # 32 (sequence, head) pairs do not fill the GPU
    assert it[:, 0].tolist() == sorted(it[:, 0].tolist()), "a uniform batch is scheduled as it comes"
    assert ws == 4 * 32 * 1 * max_parts * (128 + 2) * 4
    it, parts, max_parts, ws = _planned(st, lens, partition=4224)
    assert parts.tolist() == [1, 1, 1, 1] and max_parts == 1 and ws == 0
    assert it[:, 3].tolist() == [0] * 4 and it[:, 4].tolist() == [-1] * 4 and it[:, 5].tolist() == [4] * 4


def test_plan_attention_multi_round_batch_is_cut_and_sorted_longest_first():
    st = _state(batch=6, max_len=20000, blocks=2200)
    lens = np.array([100, 5000, 16385, 300, 2000, 9000])
    it, parts, max_parts, _ = _planned(st, lens, hq=64, hkv=64, partition=2048)   # 64 heads: 8 slots per head < 18 partitions
    _check_cover(it, parts, lens, st.table)
    assert parts.tolist() == np.maximum(1, -(-lens // 2048)).tolist() and max_parts == 9
    sizes = (lens / parts)[it[:, 0]]
    assert (np.diff(sizes) <= 1e-9).all(), "longest partitions first"


def test_plan_attention_single_round_batch_gets_even_partitions():
    st = _state(batch=5, max_len=9000, blocks=1500)
    lens = np.array([1024, 8192, 4000, 2500, 6000])
    it, parts, max_parts, _ = _planned(st, lens, hq=32, hkv=32)                    # 32 heads: 16 slots per head
    _check_cover(it, parts, lens, st.table)
    assert parts.sum() == 16 and max_parts == parts.max()
    assert (lens / parts).max() <= 1.6 * lens.sum() / 16
    st2 = _state(batch=2, max_len=1024, blocks=128)
    _, parts, _, _ = _planned(st2, [300, 700], hq=8, hkv=8)                        # never below 256 tokens per partition
    assert parts.tolist() == [1, 2]


def test_plan_attention_keeps_a_plan_while_lengths_stay_in_their_buckets_and_the_table_is_unchanged():
    st = _state(batch=3, max_len=4096, blocks=800)
    lens = np.array([1000, 3000, 130], dtype=np.int64)
    st.ensure_capacity(lens + 200)
    first = st.plan_attention(lens, 32, 8, 128, 1, False, 0)
    assert st.plan_attention(lens + 5, 32, 8, 128, 1, False, 0)[0] is first[0]      # same 64-token buckets
    assert st.plan_attention(lens + 64, 32, 8, 128, 1, False, 0)[0] is not first[0]
    again = st.plan_attention(lens, 32, 8, 128, 1, False, 0)
    st.evict(1, [3], lens)                                                           # a table entry below the lengths moved
    lens2 = lens.copy(); lens2[1] -= 16
    moved = st.plan_attention(lens, 32, 8, 128, 1, False, 0)
    assert moved[0] is not again[0]
    it = moved[0].numpy().reshape(-1, 16)
    rows = it[(it[:, 0] == 1) & (it[:, 3] == 0)]
    assert rows[0, 8:16].tolist() == st.table[1, :8].tolist()


def test_plan_attention_accepts_partitions_of_any_length_and_reports_a_short_capacity():
    from pace_mi355 import _native as nat

    st = _state(batch=1, max_len=40000, blocks=2600)
    it, parts, max_parts, ws = _planned(st, [40000], partition=65536)               # one partition of 1250 units
    assert parts.tolist() == [1] and max_parts == 1 and it[0, 3:6].tolist() == [0, -1, 4]
    lens = np.array([40000], dtype=np.int32)
    plan = nat.AttnPlan()
    out = np.zeros((2, 16), dtype=np.int32)
    sp = np.zeros(1, dtype=np.int32)
    rc = nat.load().pace_paged_attn_plan(lens.ctypes.data, st.table.ctypes.data, st.table.shape[1], 1, 32, 8, 128, 1, 0, 1024,
                                         out.ctypes.data, 2, sp.ctypes.data, ctypes.byref(plan))
    assert rc == -1 and b"do not fit the capacity" in nat.load().pace_kv_last_error() and plan.n_work_items == 40


@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_cache_histories_keep_every_sequence_intact(seed):
    """Random appends, rollbacks, evictions, compactions and beam forks driven the way PagedKVCache
    drives them, with the pool emulated on the host (one tag per token, block copies applied as
    planned): after every step the tokens read back through the table are each sequence's own
    tokens in order, and the reference counts and the free list agree with the tables."""
    from pace_mi355.llm.paged import BLOCK, PagedState

    rng = np.random.default_rng(seed)
    B, num_blocks = 4, 64
    st = PagedState(B, 16 * BLOCK, num_blocks, torch.device("cpu"))
    pool = np.full((num_blocks, BLOCK), -1, dtype=np.int64)
    lens = np.zeros(B, dtype=np.int64)
    model = [[] for _ in range(B)]
    next_tag = 0

    def copy_blocks(pairs):
        if len(pairs):
            assert not set(pairs[:, 0].tolist()) & set(pairs[:, 1].tolist())
            pool[pairs[:, 1]] = pool[pairs[:, 0]]

    def check():
        refs = np.zeros(num_blocks, dtype=np.int64)
        for b in range(B):
            n = int(st.n_blocks[b])
            assert n == (lens[b] + BLOCK - 1) // BLOCK or n >= (lens[b] + BLOCK - 1) // BLOCK
            np.add.at(refs, st.table[b, :n], 1)
            got = pool[st.table[b, :n]].reshape(-1)[: int(lens[b])].tolist()
            assert got == model[b], f"sequence {b} reads {got[:8]}.. instead of {model[b][:8]}.."
        assert np.array_equal(refs, st.allocator.refs)
        free = st.allocator.free_ids()
        assert len(set(free.tolist())) == len(free) and not refs[free].any()
        assert len(free) + int((refs > 0).sum()) == num_blocks

    for step in range(300):
        op = rng.choice(["append", "append", "append", "truncate", "evict", "compact", "fork"])
        if op == "append":
            counts = rng.integers(0, 20, B)
            need = sum(int((lens[b] + counts[b] + BLOCK - 1) // BLOCK - st.n_blocks[b]) for b in range(B)) + B  # + copies
            if need > st.allocator.num_free or (lens + counts).max() > 16 * BLOCK:
                continue
            if st.tails_dirty:
                copy_blocks(st.unshare_tails(lens))
            st.ensure_capacity(lens + counts)
            width = int(counts.max(initial=0))
            if width:
                slots = st.slots(lens, counts, width)
                for b in range(B):
                    for t in range(int(counts[b])):
                        pool[slots[b, t] // BLOCK, slots[b, t] % BLOCK] = next_tag
                        model[b].append(next_tag)
                        next_tag += 1
                    assert (slots[b, int(counts[b]):] == -1).all()
            lens = lens + counts
        elif op == "truncate":
            remove = np.minimum(rng.integers(0, 24, B), lens)
            lens = lens - remove
            for b in range(B):
                del model[b][int(lens[b]):]
            if remove.any():
                st.release_beyond(lens)
                st.lengths_shrank()
        elif op == "evict":
            b = int(rng.integers(0, B))
            n = int(st.n_blocks[b])
            if n == 0:
                continue
            drop = sorted(set(rng.integers(0, n, rng.integers(1, 3)).tolist()))
            keep = [t for j in range(n) if j not in drop for t in model[b][j * BLOCK:(j + 1) * BLOCK]]
            lens = st.evict(b, drop, lens)
            st.lengths_shrank()
            model[b] = keep
        elif op == "compact":
            moves = st.plan_compaction()
            copy_blocks(moves)
            st.apply_moves(moves)
            live = st.live_block_count()
            used = np.unique(np.concatenate([st.table[b, : int(st.n_blocks[b])] for b in range(B)]))
            assert used.size == live and (used.size == 0 or used.max() == live - 1)
        else:
            src = rng.integers(0, B, B).tolist()
            st.fork(src)
            lens = lens[src].copy()
            model = [list(model[i]) for i in src]
        check()
    assert next_tag > 500  # the history really appended
