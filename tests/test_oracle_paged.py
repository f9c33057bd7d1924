"""Pin the paged oracle: it must equal a replay of the surviving tokens through the
contiguous reference cache, and its slot arithmetic must equal numpy indexing."""
import numpy as np
import pytest
import torch

from oracle.cache_ref import DynamicKVCacheRef
from oracle.paged_ref import RaggedCacheModel, copy_blocks_np, gather_slots, scatter_slots, slots_for


def test_ragged_model_equals_dynamic_cache_replay_per_sequence():
    rng = np.random.default_rng(0)
    B, H, D = 3, 2, 4
    model = RaggedCacheModel(B, H, D, dtype=torch.float32)
    replay = [DynamicKVCacheRef(0) for _ in range(B)]
    g = torch.Generator().manual_seed(1)
    for _ in range(5):
        T = int(rng.integers(1, 20))
        counts = rng.integers(0, T + 1, size=B)
        k, v = torch.randn(B, H, T, D, generator=g), torch.randn(B, H, T, D, generator=g)
        model.append(k, v, counts)
        for b in range(B):
            if counts[b]:
                replay[b].update_cache(k[b : b + 1, :, : counts[b]], v[b : b + 1, :, : counts[b]], 2)
    rem = [2, 0, 1]
    model.truncate(rem)
    for b in range(B):
        replay[b].remove_cache(rem[b])
    for b in range(B):
        assert torch.equal(model.k[b], replay[b].key[0]) and torch.equal(model.v[b], replay[b].value[0])
    with pytest.raises(ValueError, match="Cannot remove more tokens"):
        model.truncate([10_000, 0, 0])


def test_evict_keeps_survivors_in_order():
    model = RaggedCacheModel(1, 1, 1, dtype=torch.float32)
    x = torch.arange(40, dtype=torch.float32).view(1, 1, 40, 1)
    model.append(x, x)
    model.evict_blocks(0, [0, 2], 16)  # tokens 0-15 and 32-39 go
    assert model.k[0].flatten().tolist() == list(range(16, 32))
    K, _ = model.dense(n_rep=2, pad_to=20)
    assert K.shape == (1, 2, 20, 1) and K[0, 1, :16, 0].tolist() == list(range(16, 32)) and K[0, 0, 16:].sum() == 0


def test_slot_functions_are_numpy_indexing():
    rng = np.random.default_rng(3)
    table = rng.permutation(12).astype(np.int32).reshape(3, 4)
    rows = np.zeros((12 * 16, 2), dtype=np.float32)
    lens = [40, 64, 7]
    want = []
    for b, n in enumerate(lens):
        new = rng.standard_normal((n, 2)).astype(np.float32)
        want.append(new)
        s = slots_for(table, b, 0, n, 16)
        assert s[0] == table[b, 0] * 16 and (n <= 16 or s[16] == table[b, 1] * 16)
        scatter_slots(rows, new, s)
    dense = gather_slots(rows, table, lens, 16, 64)
    for b, n in enumerate(lens):
        assert np.array_equal(dense[b, :n], want[b]) and not dense[b, n:].any()
    scatter_slots(rows, np.ones((2, 2), np.float32), np.array([-1, -5]))  # negative slots are padding


def test_copy_blocks_np():
    pool = np.arange(6 * 3).reshape(6, 3).copy()
    copy_blocks_np(pool, np.array([[4, 0], [5, 2]]))
    assert pool[0].tolist() == [12, 13, 14] and pool[2].tolist() == [15, 16, 17]
    with pytest.raises(AssertionError):
        copy_blocks_np(pool, np.array([[1, 2], [2, 3]]))


def test_model_attention_uses_per_row_causal_limit():
    model = RaggedCacheModel(1, 1, 2, dtype=torch.float32)
    k = torch.tensor([[[[1.0, 0.0], [0.0, 1.0], [1.0, 1.0]]]])
    v = torch.tensor([[[[1.0, 0.0], [0.0, 1.0], [5.0, 5.0]]]])
    model.append(k, v)
    q = torch.zeros(1, 1, 2, 2)  # uniform scores: each row averages what it may read
    out = model.attention(q, 1)
    assert torch.allclose(out[0, 0, 0], torch.tensor([0.5, 0.5]))  # row 0 reads tokens 0..1
    assert torch.allclose(out[0, 0, 1], torch.tensor([2.0, 2.0]))  # row 1 reads tokens 0..2
