"""Pins ``oracle/rope_ref.py`` (the reference has no test of its rotary embedding).

Independent sources: complex multiplication in float64, invariants of a rotation, an
integer-bit emulation of bf16 rounding, and the inverse frequencies of the installed
``transformers`` for the scaled variants.
"""
import math

import numpy as np
import pytest
import torch

from oracle import rope_ref


def _complex_rotate(x, pos, freq, neox):
    """x [B,H,S,D] float64, pos [B,S], freq [D/2] -> rotation by e^{i pos w} on the pairs."""
    B, H, S, D = x.shape
    ang = pos[:, None, :, None].astype(np.float64) * freq[None, None, None, :].astype(np.float64)
    ph = np.exp(1j * ang)
    if neox:
        z = x[..., : D // 2] + 1j * x[..., D // 2:]
        z = z * ph
        return np.concatenate([z.real, z.imag], axis=-1)
    z = x[..., 0::2] + 1j * x[..., 1::2]
    z = z * ph
    out = np.empty_like(x)
    out[..., 0::2], out[..., 1::2] = z.real, z.imag
    return out


@pytest.mark.parametrize("neox", [True, False])
def test_rotate_is_complex_multiplication(neox):
    torch.manual_seed(0)
    B, H, S, D = 2, 3, 7, 16
    x = torch.randn(B, H, S, D, dtype=torch.float32)
    pos = torch.randint(0, 50, (B, S))
    cos, sin, kind, rot = rope_ref.cos_sin_tables(None, D, 64, 10000.0)
    assert kind == "default" and rot == D and cos.shape == (64, D // 2)
    c, s = rope_ref.lookup(cos, sin, pos, torch.float32)
    got = rope_ref.rotate(x, c, s, neox=neox).double().numpy()
    freq = 1.0 / (10000.0 ** (np.arange(0, D, 2) / D))
    want = _complex_rotate(x.double().numpy(), pos.numpy(), freq, neox)
    np.testing.assert_allclose(got, want, atol=2e-5)


def test_default_table_closed_form():
    cos, sin, _, _ = rope_ref.cos_sin_tables(None, 8, 32, 10000.0)
    for p in (0, 1, 17, 31):
        for i in range(4):
            w = 10000.0 ** (-2 * i / 8)
            assert abs(cos[p, i].item() - math.cos(p * w)) < 1e-5
            assert abs(sin[p, i].item() - math.sin(p * w)) < 1e-5
    assert torch.all(cos[0] == 1) and torch.all(sin[0] == 0)


@pytest.mark.parametrize("neox", [True, False])
def test_rotation_invariants(neox):
    torch.manual_seed(1)
    D = 32
    cos, sin, _, _ = rope_ref.cos_sin_tables(None, D, 256, 10000.0)
    q = torch.randn(1, 1, 1, D, dtype=torch.float64)
    k = torch.randn(1, 1, 1, D, dtype=torch.float64)
    cos, sin = cos.double(), sin.double()

    def at(x, p):
        c, s = rope_ref.lookup(cos, sin, torch.tensor([[p]]), torch.float64)
        return rope_ref.rotate(x, c, s, neox=neox)

    # position 0 is the identity; norms are preserved; q_m . k_n depends on m - n only
    assert torch.equal(at(q, 0), q)
    assert abs(at(q, 123).norm().item() - q.norm().item()) < 1e-6
    d1 = (at(q, 40) * at(k, 10)).sum().item()
    d2 = (at(q, 130) * at(k, 100)).sum().item()
    assert abs(d1 - d2) < 1e-5
    # a wrong sign (rotating k the other way) breaks the relative-position property
    d3 = (at(q, 40) * at(k, 70)).sum().item()
    assert abs(d1 - d3) > 1e-3


def _rne_bf16(a32: np.ndarray) -> np.ndarray:
    """float32 -> bf16 (round to nearest even) -> float32, with integer arithmetic only."""
    bits = a32.astype(np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32)


@pytest.mark.parametrize("neox", [True, False])
def test_bf16_rounding_sequence(neox):
    """bf16 activations: every product and the sum are rounded separately (three roundings)."""
    torch.manual_seed(2)
    B, H, S, D = 2, 2, 5, 16
    x = torch.randn(B, H, S, D).to(torch.bfloat16)
    pos = torch.randint(0, 200, (B, S))
    cos, sin, _, _ = rope_ref.cos_sin_tables(None, D, 256, 10000.0)
    c, s = rope_ref.lookup(cos, sin, pos, torch.bfloat16)
    got = rope_ref.rotate(x, c, s, neox=neox).float().numpy()
    xf = x.float().numpy()
    cf = _rne_bf16(cos.numpy())[pos.numpy()][:, None]
    sf = _rne_bf16(sin.numpy())[pos.numpy()][:, None]
    x1, x2 = (xf[..., : D // 2], xf[..., D // 2:]) if neox else (xf[..., 0::2], xf[..., 1::2])
    o1 = _rne_bf16(_rne_bf16(x1 * cf) - _rne_bf16(x2 * sf))
    o2 = _rne_bf16(_rne_bf16(x2 * cf) + _rne_bf16(x1 * sf))
    want = np.concatenate([o1, o2], -1) if neox else np.stack([o1, o2], -1).reshape(B, H, S, D)
    np.testing.assert_array_equal(got, want)
    # a fused multiply-add (one rounding) gives different bits somewhere: the order matters
    fused = _rne_bf16(x1 * cf - x2 * sf)
    assert np.any(fused != o1)


def test_longrope_form_equals_neox_form_and_passes_tail_through():
    torch.manual_seed(3)
    B, H, S, D, rot = 1, 2, 4, 32, 16
    x = torch.randn(B, H, S, D).to(torch.bfloat16)
    cos, sin, _, _ = rope_ref.cos_sin_tables(None, rot, 64, 10000.0)
    c, s = rope_ref.lookup(cos, sin, torch.tensor([[3, 9, 27, 63]]), torch.bfloat16)
    a = rope_ref.rotate(x, c, s, neox=True, rotary_dim=rot)
    b = rope_ref.rotate_longrope_form(x, c, s, rot)
    assert torch.equal(a, b)
    assert torch.equal(a[..., rot:], x[..., rot:])


def _hf_inv_freq(kind, params, head_dim, max_pos, seq_len=None):
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS

    cfg = LlamaConfig(hidden_size=head_dim * 2, num_attention_heads=2, max_position_embeddings=max_pos,
                      rope_parameters=dict(rope_type=kind, **params))
    f, amp = ROPE_INIT_FUNCTIONS[kind](cfg, torch.device("cpu"), seq_len=seq_len)
    return f.float(), amp


def _table_freq(cos, sin):
    """Recover the frequencies from row 1 of a table (angle = 1 * w)."""
    return torch.atan2(sin[1], cos[1])


def test_llama3_table_matches_transformers():
    params = dict(rope_theta=500000.0, factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                  original_max_position_embeddings=8192)
    want, amp = _hf_inv_freq("llama3", params, 128, 131072)
    scaling = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0,
                   original_max_position_embeddings=8192)
    got = rope_ref.llama3_freq(500000.0, 128, 8.0, 1.0, 4.0, 8192)
    assert amp == 1.0
    torch.testing.assert_close(got, want, rtol=1e-6, atol=0)
    cos, sin, kind, _ = rope_ref.cos_sin_tables(scaling, 128, 64, 500000.0)
    assert kind == "llama3"
    torch.testing.assert_close(_table_freq(cos, sin), want, rtol=1e-5, atol=1e-7)


def test_dynamic_table_matches_transformers_at_full_length():
    s, D, max_pos = 2.0, 64, 128
    want, _ = _hf_inv_freq("dynamic", dict(rope_theta=10000.0, factor=s), D, max_pos, seq_len=int(max_pos * s))
    cos, sin, _, _ = rope_ref.cos_sin_tables(dict(rope_type="dynamic", scaling_factor=s), D, max_pos, 10000.0)
    assert cos.shape[0] == int(max_pos * s)
    torch.testing.assert_close(_table_freq(cos, sin), want, rtol=1e-5, atol=1e-7)


def test_longrope_tables_match_transformers():
    D, orig, max_pos = 32, 64, 256
    short = [1.0 + 0.01 * i for i in range(D // 2)]
    long_ = [2.0 + 0.1 * i for i in range(D // 2)]
    scaling = dict(rope_type="longrope", short_factor=short, long_factor=long_)
    cos, sin, kind, _ = rope_ref.cos_sin_tables(scaling, D, max_pos, 10000.0, original_max_position_embeddings=orig)
    assert kind == "longrope" and cos.shape[0] == orig + max_pos
    amp = math.sqrt(1 + math.log(max_pos / orig) / math.log(orig))
    params = dict(rope_theta=10000.0, short_factor=short, long_factor=long_, factor=max_pos / orig,
                  original_max_position_embeddings=orig)
    f_short, a1 = _hf_inv_freq("longrope", params, D, max_pos, seq_len=orig)
    f_long, a2 = _hf_inv_freq("longrope", params, D, max_pos, seq_len=max_pos)
    assert abs(a1 - amp) < 1e-6 and abs(a2 - amp) < 1e-6
    # row 1 of each half: amplitude * (cos w, sin w)
    torch.testing.assert_close(torch.atan2(sin[1], cos[1]), f_short, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(torch.atan2(sin[orig + 1], cos[orig + 1]), f_long, rtol=1e-5, atol=1e-7)
    torch.testing.assert_close(torch.hypot(cos[orig + 1], sin[orig + 1]), torch.full((D // 2,), amp), rtol=1e-5, atol=0)


def test_linear_scales_the_amplitude_like_the_reference():
    # pace/ops/rotary_embedding.py:119-130 hands the factor to the cos / sin multiplier
    # (not to the positions, as transformers does): restated as it is written.
    base_c, base_s, _, _ = rope_ref.cos_sin_tables(None, 16, 32, 10000.0)
    cos, sin, _, _ = rope_ref.cos_sin_tables(dict(type="linear", scaling_factor=4.0), 16, 32, 10000.0)
    assert torch.equal(cos, base_c * 4.0) and torch.equal(sin, base_s * 4.0)


def test_partial_rotary_and_unknown_type():
    cos, _, _, rot = rope_ref.cos_sin_tables(None, 64, 16, 10000.0, partial_rotary_factor=0.5)
    assert rot == 32 and cos.shape == (16, 16)
    with pytest.raises(AssertionError, match="Unsupported RoPE type"):
        rope_ref.cos_sin_tables(dict(rope_type="yarn"), 64, 16, 10000.0)


def test_longrope_row_selection():
    ids = torch.tensor([[0, 1, 2], [5, 6, 7]])
    assert torch.equal(rope_ref.longrope_rows(ids, 8), ids)
    ids2 = torch.tensor([[0, 1, 2], [7, 8, 9]])
    assert torch.equal(rope_ref.longrope_rows(ids2, 8), ids2 + 8)


def test_longrope_selection_agrees_with_transformers_off_the_boundary():
    """transformers switches to the long factors when ``max(position_ids) + 1`` exceeds the original
    length (``dynamic_rope_update`` of modeling_rope_utils); the reference when any id exceeds it
    (``rotary_embedding.py:381-385``).  The two rules agree except for a batch whose largest id is
    exactly the original length: checked here on both sides of that single point, and at the point
    the oracle follows the reference as written."""
    D, orig, max_pos = 32, 64, 256
    short = [1.0 + 0.01 * i for i in range(D // 2)]
    long_ = [2.0 + 0.1 * i for i in range(D // 2)]
    scaling = dict(rope_type="longrope", short_factor=short, long_factor=long_)
    cos, sin, _, _ = rope_ref.cos_sin_tables(scaling, D, max_pos, 10000.0, original_max_position_embeddings=orig)
    params = dict(rope_theta=10000.0, short_factor=short, long_factor=long_, factor=max_pos / orig,
                  original_max_position_embeddings=orig)
    for top in (3, orig - 1, orig + 1, max_pos - 1):
        ids = torch.tensor([[0, 1, top]])
        rows = rope_ref.longrope_rows(ids, orig)
        f_hf, _ = _hf_inv_freq("longrope", params, D, max_pos, seq_len=top + 1)  # the library's choice for this batch
        got = torch.atan2(sin[rows[0, 1]], cos[rows[0, 1]])                       # angle of position 1 = its frequency
        torch.testing.assert_close(got, f_hf, rtol=1e-5, atol=1e-7)
    # the one point where the rules differ: largest id == original length -> the reference stays short
    assert torch.equal(rope_ref.longrope_rows(torch.tensor([[0, orig]]), orig), torch.tensor([[0, orig]]))
