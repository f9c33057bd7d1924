"""Pin the cache oracle: the reference's own test expectations
(tests/llm_infra/test_cache.py of the reference) and closed forms."""
import math

import pytest
import torch

from oracle.cache_ref import (
    BMCKVCacheRef,
    CacheKind,
    DynamicKVCacheRef,
    KVCacheManagerRef,
    cache_class_for,
    repeat_kv,
    valid_prefix,
)


class MockConfig:
    num_hidden_layers = 2


# ---- expectations the reference's tests hold (tests/llm_infra/test_cache.py:30-80) ----
def test_reference_manager_expectations():
    mgr = KVCacheManagerRef(MockConfig(), 128, CacheKind.DYNAMIC)
    assert len(mgr.cache_objects) == 2
    assert isinstance(mgr[0], DynamicKVCacheRef)
    assert mgr.update_mask(torch.ones(2, 10), 10).shape == (2, 10)


def test_reference_bmc_expectations():
    bmc = BMCKVCacheRef(128)
    k, v = bmc.update_cache(torch.rand(2, 10, 64), torch.rand(2, 10, 64), concat_dim=1)
    assert k.shape[1] == 11 and v.shape[1] == 11  # 128 // int(sqrt(128)) = 11 tokens per split
    assert bmc.update_mask(torch.ones(2, 10), 10).shape == (2, 11)


def test_reference_dynamic_expectations():
    dyn = DynamicKVCacheRef(128)
    k, v = dyn.update_cache(torch.rand(2, 10, 64), torch.rand(2, 10, 64), concat_dim=1)
    assert k.shape[1] == 10 and v.shape[1] == 10


# ---- closed forms ----
@pytest.mark.parametrize("cls", [DynamicKVCacheRef, BMCKVCacheRef])
def test_append_is_concatenation(cls):
    g = torch.Generator().manual_seed(0)
    cache = cls(300)
    parts_k, parts_v = [], []
    for T in (17, 1, 1, 40, 3, 1):
        k = torch.randn(2, 4, T, 8, generator=g)
        v = torch.randn(2, 4, T, 8, generator=g)
        parts_k.append(k)
        parts_v.append(v)
        cache.update_cache(k, v, 2)
        lk, lv = valid_prefix(cache)
        assert torch.equal(lk, torch.cat(parts_k, 2)) and torch.equal(lv, torch.cat(parts_v, 2))
        assert cache.seq_len == sum(p.shape[2] for p in parts_k)


@pytest.mark.parametrize("max_len,tps", [(128, 11), (576, 24), (4224, 66), (2048, 45)])
def test_bmc_split_arithmetic(max_len, tps):
    assert BMCKVCacheRef(max_len).tokens_per_split == tps == max_len // int(math.sqrt(max_len))


def test_bmc_env_override(monkeypatch):
    monkeypatch.setenv("PACE_BMC_NUM_SPLITS", "4")
    assert BMCKVCacheRef(128).tokens_per_split == 32


def test_bmc_capacity_padding_and_regrow_rule():
    bmc = BMCKVCacheRef(128)  # 11 tokens per split
    k = torch.ones(1, 1, 11, 2)
    K, _ = bmc.update_cache(k, k, 2)
    assert K.shape[2] == 11  # exactly full: holds, no padding
    K, _ = bmc.update_cache(k[:, :, :1], k[:, :, :1], 2)
    assert K.shape[2] == 22 and bmc.seq_len == 12
    assert torch.count_nonzero(K[:, :, 12:]) == 0  # tail rows are zeros
    for _ in range(10):  # reaching 22 re-makes a buffer of the same 22 rows (">=" rule) -- contents survive
        K, _ = bmc.update_cache(k[:, :, :1], k[:, :, :1], 2)
    assert bmc.seq_len == 22 and K.shape[2] == 22 and torch.count_nonzero(K) == K.numel()
    assert bmc.update_mask(torch.zeros(1, 1, 1, 22), 22).shape[-1] == 22
    m = bmc.update_mask(torch.zeros(1, 1, 1, 23, dtype=torch.bfloat16), 23)
    assert m.shape[-1] == 33 and (m[..., 23:] == torch.finfo(torch.bfloat16).min).all()


def test_bmc_rollback_leaves_stale_rows_and_is_overwritten():
    bmc = BMCKVCacheRef(128)
    a = torch.arange(1, 6, dtype=torch.float32).view(1, 1, 5, 1)
    bmc.update_cache(a, a, 2)
    bmc.remove_cache(2)
    assert bmc.seq_len == 3 and bmc.key[0, 0, 3, 0] == 4  # stale row still there
    b = torch.full((1, 1, 1, 1), 9.0)
    K, _ = bmc.update_cache(b, b, 2)
    assert K[0, 0, :5, 0].tolist() == [1, 2, 3, 9, 5]


@pytest.mark.parametrize("cls", [DynamicKVCacheRef, BMCKVCacheRef])
def test_truncate_prefix_and_errors(cls):
    cache = cls(64)
    cache.remove_cache(5)  # empty cache: silently nothing (reference guards on key is None)
    k = torch.randn(2, 2, 9, 4)
    cache.update_cache(k, k, 2)
    cache.remove_cache(4)
    lk, _ = valid_prefix(cache)
    assert torch.equal(lk, k[:, :, :5])
    with pytest.raises(ValueError, match="Cannot remove more tokens than available in cache."):
        cache.remove_cache(6)
    with pytest.raises(AssertionError, match="concat_dim should be the same for all updates"):
        cache.update_cache(k, k, 1)


def test_beam_reorder_is_index_select():
    dyn = DynamicKVCacheRef(32)
    k = torch.randn(4, 2, 5, 3)
    dyn.update_cache(k, k.clone(), 2)
    idx = torch.tensor([3, 3, 0, 1])
    dyn.update_cache_with_beam_indices(idx)
    assert torch.equal(dyn.key, k[idx])


def test_repeat_kv_is_repeat_interleave():
    x = torch.randn(2, 3, 5, 4)
    out = repeat_kv(x, 4)
    assert out.shape == (2, 12, 5, 4)
    for h in range(12):
        assert torch.equal(out[:, h], x[:, h // 4])
    assert repeat_kv(x, 1) is x


def test_kind_parsing():
    assert cache_class_for("dynamic") is DynamicKVCacheRef and cache_class_for("bmc") is BMCKVCacheRef
    with pytest.raises(ValueError):
        cache_class_for("paged-nope")


def test_manager_remove_and_len():
    mgr = KVCacheManagerRef(MockConfig(), 64, "bmc")
    k = torch.randn(1, 1, 6, 2)
    for layer in range(2):
        mgr[layer].update_cache(k, k, 2)
    assert len(mgr) == 6
    mgr.remove_cache(2)
    assert len(mgr) == 4 and mgr[1].seq_len == 4
