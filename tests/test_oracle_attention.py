"""Pin the attention oracle against what the mathematics fixes."""
import math
import warnings

import numpy as np
import pytest
import torch

from oracle.attention_ref import (
    causal_mask_4d,
    check_attention_args,
    lengths_mask_4d,
    sdpa_bruteforce_f64,
    sdpa_fp32,
    sdpa_jit_emulated,
    sdpa_native,
)
from oracle.cache_ref import repeat_kv


def _rand(shape, seed, dtype=torch.float32):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


@pytest.mark.parametrize("B,N,S,H,L,mask_s", [(1, 1, 1, 1, 1, 1), (2, 3, 2, 5, 7, 1), (1, 2, 3, 4, 6, 3)])
def test_fp32_matches_bruteforce_f64(B, N, S, H, L, mask_s):
    q, k, v = _rand((B, N, S, H), 1), _rand((B, N, L, H), 2), _rand((B, N, L, H), 3)
    m = _rand((B, 1, mask_s, L), 4)
    want = sdpa_bruteforce_f64(q, k, v, m)
    for fn in (sdpa_fp32, sdpa_native, sdpa_jit_emulated):
        np.testing.assert_allclose(fn(q, k, v, m).double().numpy(), want, atol=2e-6, rtol=2e-6)


def test_transposed_operand_or_dropped_scale_would_fail():
    # H != L and S != L so that a transposed K, a missing 1/sqrt(H) or a mask on the wrong axis changes the result
    q, k, v, m = _rand((1, 1, 2, 9), 5), _rand((1, 1, 4, 9), 6), _rand((1, 1, 4, 9), 7), _rand((1, 1, 1, 4), 8)
    want = sdpa_bruteforce_f64(q, k, v, m)
    logits = (q.double() @ k.double().transpose(-1, -2)).numpy()  # no scale
    w = np.exp(logits + m.double().numpy())
    w /= w.sum(-1, keepdims=True)
    wrong = w @ v.double().numpy()
    assert np.abs(wrong - want).max() > 1e-3


def test_single_key_returns_value_row():
    q, k, v = _rand((2, 2, 3, 8), 1), _rand((2, 2, 1, 8), 2), _rand((2, 2, 1, 8), 3)
    out = sdpa_fp32(q, k, v, torch.zeros(2, 1, 1, 1))
    assert torch.allclose(out, v.expand(-1, -1, 3, -1), atol=1e-6)


def test_mask_row_shift_invariance_and_key_permutation():
    q, k, v = _rand((1, 2, 2, 8), 1), _rand((1, 2, 6, 8), 2), _rand((1, 2, 6, 8), 3)
    m = _rand((1, 1, 2, 6), 4)
    base = sdpa_fp32(q, k, v, m)
    assert torch.allclose(sdpa_fp32(q, k, v, m + 3.25), base, atol=1e-5)
    perm = torch.tensor([4, 0, 5, 2, 1, 3])
    assert torch.allclose(sdpa_fp32(q, k[:, :, perm], v[:, :, perm], m[..., perm]), base, atol=1e-5)


def test_uniform_scores_average_values():
    k = torch.zeros(1, 1, 5, 4)
    v = _rand((1, 1, 5, 4), 3)
    out = sdpa_fp32(_rand((1, 1, 1, 4), 1), k, v, torch.zeros(1, 1, 1, 5))
    assert torch.allclose(out[0, 0, 0], v[0, 0].mean(0), atol=1e-6)


def test_gqa_equivalence():
    """attention over repeat_kv-expanded heads == per-KV-head attention of the grouped queries."""
    n_rep, hkv = 4, 2
    q = _rand((2, hkv * n_rep, 1, 16), 1)
    k, v = _rand((2, hkv, 9, 16), 2), _rand((2, hkv, 9, 16), 3)
    full = sdpa_fp32(q, repeat_kv(k, n_rep), repeat_kv(v, n_rep), torch.zeros(2, 1, 1, 9))
    for h in range(hkv * n_rep):
        one = sdpa_fp32(q[:, h : h + 1], k[:, h // n_rep : h // n_rep + 1], v[:, h // n_rep : h // n_rep + 1], torch.zeros(2, 1, 1, 9))
        assert torch.allclose(full[:, h : h + 1], one, atol=1e-6)


def test_jit_emulation_within_reference_bf16_tolerance():
    """The reference accepts 1e-1 between its op and torch in bf16 (tests/ops/test_sdpa.py:113-127)."""
    q, k, v = _rand((2, 4, 8, 64), 1, torch.bfloat16), _rand((2, 4, 128, 64), 2, torch.bfloat16), _rand((2, 4, 128, 64), 3, torch.bfloat16)
    m = _rand((2, 1, 1, 128), 4, torch.bfloat16)
    a, b = sdpa_jit_emulated(q, k, v, m).float(), sdpa_native(q, k, v, m).float()
    assert a.dtype == torch.float32 and sdpa_jit_emulated(q, k, v, m).dtype == torch.bfloat16
    assert torch.allclose(a, b, atol=1e-1, rtol=1e-1)
    assert torch.allclose(a, sdpa_fp32(q, k, v, m), atol=2e-2, rtol=2e-2)


def test_causal_mask_closed_form_small():
    m2 = torch.tensor([[0, 0, 1, 1, 1], [1, 1, 1, 1, 1]])
    got = causal_mask_4d(m2, 2, 5, torch.float32)
    lo = torch.finfo(torch.float32).min
    want = torch.tensor(
        [[[[lo, lo, 0, 0, lo], [lo, lo, 0, 0, 0]]], [[[0, 0, 0, 0, lo], [0, 0, 0, 0, 0]]]], dtype=torch.float32
    )
    assert torch.equal(got, want)


@pytest.mark.parametrize("q_len,kv_len,dtype", [(1, 9, torch.float32), (4, 9, torch.bfloat16), (9, 9, torch.float32)])
def test_causal_mask_against_installed_transformers(q_len, kv_len, dtype):
    """The reference calls transformers' AttentionMaskConverter.to_4d (llama.py:292-299, release 4.51.3);
    the class of the same name in the installed release must agree with the closed form."""
    try:
        from transformers.modeling_attn_mask_utils import AttentionMaskConverter
    except Exception:
        pytest.skip("transformers' AttentionMaskConverter not importable")
    g = torch.Generator().manual_seed(q_len * 100 + kv_len)
    pad = torch.randint(0, 4, (3,), generator=g)
    m2 = torch.ones(3, kv_len, dtype=torch.long)
    for b, p in enumerate(pad.tolist()):
        m2[b, :p] = 0
    with warnings.catch_warnings():
        warnings.simplefilter("ignore")
        want = AttentionMaskConverter(is_causal=True, sliding_window=None).to_4d(m2, q_len, key_value_length=kv_len, dtype=dtype)
    assert torch.equal(causal_mask_4d(m2, q_len, kv_len, dtype), want)


def test_lengths_mask_equals_causal_mask_of_right_padded_batch():
    lens = [5, 9, 1]
    for S in (1, 3):
        got = lengths_mask_4d(lens, S, 9, torch.float32)
        for b, n in enumerate(lens):
            if n < S:
                continue
            m2 = torch.ones(1, n, dtype=torch.long)
            want = causal_mask_4d(m2, S, n, torch.float32)
            assert torch.equal(got[b : b + 1, :, :, :n], want)
            assert (got[b, :, :, n:] == torch.finfo(torch.float32).min).all()


def test_argument_checks_follow_reference_order_and_text():
    q = torch.zeros(2, 2, 3, 4)
    k = torch.zeros(2, 2, 5, 4)
    m = torch.zeros(2, 1, 1, 5)
    assert check_attention_args(q, k, k, m, None) == 0
    assert check_attention_args(q, k, k, m, True) == 1
    with pytest.raises(RuntimeError, match="attention requires 4D inputs"):
        check_attention_args(q.view(4, 3, 4), k, k, m, 0)
    with pytest.raises(RuntimeError, match="attention requires 4D inputs"):
        check_attention_args(q, k, k, m.view(2, 5), 0)
    with pytest.raises(RuntimeError, match="requires Key and Value sizes to be of same shape"):
        check_attention_args(q, k, torch.zeros(2, 2, 6, 4), m, 0)
    with pytest.raises(RuntimeError, match="only support the dtypes Float and BF16 types for input"):
        check_attention_args(q.to(torch.int8), k, k, m, 0)
    with pytest.raises(RuntimeError, match="attention requires use_KQ to be 0 or 1"):
        check_attention_args(q, k, k, m, 7)
    # order: dims before K/V shape before dtype before use_KQ
    with pytest.raises(RuntimeError, match="4D inputs"):
        check_attention_args(q.view(4, 3, 4).to(torch.int8), k, torch.zeros(1), m, 9)
    with pytest.raises(RuntimeError, match="same shape"):
        check_attention_args(q.to(torch.int8), k, torch.zeros(2, 2, 6, 4), m, 9)
    with pytest.raises(RuntimeError, match="dtypes Float and BF16"):
        check_attention_args(q.to(torch.int8), k, k, m, 9)
