"""The committed fixtures of tests/golden: the oracle must still reproduce them (CPU), and the
HIP path must match them (GPU; bit-exact for cache and rotary rows, tolerance for attention)."""
import importlib.util
import os

import numpy as np
import pytest
import torch

from helpers import assert_attention_close, assert_bits_equal

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _load(name):
    return np.load(os.path.join(GOLDEN, name), allow_pickle=False)


def _bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)


def test_oracle_reproduces_the_fixtures():
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    for name, make in mod.FIXTURES.items():
        fresh, stored = make(), _load(name)
        assert sorted(fresh) == sorted(stored.files), name
        for key in fresh:
            np.testing.assert_array_equal(np.asarray(fresh[key]), stored[key], err_msg=f"{name}:{key}")


@pytest.mark.gpu
def test_paged_cache_matches_the_cache_fixture(device):
    from pace_mi355.llm import PagedKVCache

    fx = _load("cache_append.npz")
    cache = PagedKVCache(64)
    for i, _ in enumerate(fx["steps"]):
        cache.update_cache(_bf16(fx[f"k{i}"]).to(device), _bf16(fx[f"v{i}"]).to(device), 2)
    cache.remove_cache(4)
    gk, gv = cache.gather()
    assert_bits_equal(gk, _bf16(fx["key"]), "key")
    assert_bits_equal(gv, _bf16(fx["value"]), "value")


@pytest.mark.gpu
def test_rope_matches_the_rope_fixture(device):
    import ctypes

    from pace_mi355 import _native as nat

    fx = _load("rope.npz")
    x = _bf16(fx["x"]).to(device)
    cos = torch.from_numpy(fx["cos"]).to(device).contiguous()
    sin = torch.from_numpy(fx["sin"]).to(device).contiguous()
    rows = torch.from_numpy(fx["positions"]).to(device=device, dtype=torch.int32)
    B, H, S, D = x.shape
    for style, want in ((0, "neox"), (1, "gptj")):
        out = torch.empty_like(x)
        d = nat.RopeDesc(cos=cos.data_ptr(), sin=sin.data_ptr(), table_dtype=nat.DTYPE_F32, table_rows=cos.shape[0],
                         rotary_dim=D, interleaved=style, positions=rows.data_ptr(), pos_stride_b=rows.stride(0))
        nat.check(nat.load().pace_rope_apply(ctypes.byref(d), x.data_ptr(), out.data_ptr(), x.stride(0), x.stride(1), x.stride(2), H,
                                             None, None, 0, 0, 0, 0, B, S, D, nat.current_stream_ptr()))
        assert_bits_equal(out, _bf16(fx[want]), want)


@pytest.mark.gpu
def test_paged_attention_matches_the_attention_fixture(device):
    from pace_mi355.llm import PagedKVCache

    fx = _load("paged_attention.npz")
    n_rep, lens = int(fx["n_rep"]), fx["lens"].tolist()
    k, v = _bf16(fx["k"]), _bf16(fx["v"])
    cache = PagedKVCache(64, num_kv_heads=k.shape[1], n_rep=n_rep)
    cache.append_ragged(k.to(device), v.to(device), lens)
    assert_attention_close(cache.attend(_bf16(fx["q1"]).to(device)), torch.from_numpy(fx["decode"]), "decode")
    assert_attention_close(cache.attend(_bf16(fx["q3"]).to(device)), torch.from_numpy(fx["verify"]), "verify")
