"""Host side of the rotary-embedding operator: tables and row selection against the oracle,
constructor contract, and loud failure off the GPU (no GPU needed)."""
import pytest
import torch

from oracle import rope_ref
from pace_mi355.ops import RotaryEmbedding
from pace_mi355.ops.enum import OperatorType

LLAMA3 = dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=8192)
SHORT = [1.0 + 0.01 * i for i in range(32)]
LONG = [2.0 + 0.1 * i for i in range(32)]


@pytest.mark.parametrize(
    "scaling,kwargs",
    [
        (None, {}),
        (dict(type="linear", scaling_factor=2.0), {}),
        (dict(rope_type="dynamic", scaling_factor=2.0), {}),
        (LLAMA3, {}),
        (dict(rope_type="longrope", short_factor=SHORT, long_factor=LONG), dict(original_max_position_embeddings=64)),
        (dict(rope_type="longrope", short_factor=SHORT, long_factor=LONG, attention_factor=1.25), {}),
        (None, dict(partial_rotary_factor=0.5)),
    ],
)
def test_tables_equal_the_oracle(scaling, kwargs):
    D = 64 if "partial_rotary_factor" not in kwargs else 128
    mod = RotaryEmbedding(scaling, D, 256, 10000.0, **kwargs)
    cos, sin, kind, rot = rope_ref.cos_sin_tables(
        scaling, D, 256, 10000.0, partial_rotary_factor=kwargs.get("partial_rotary_factor", 1.0),
        original_max_position_embeddings=kwargs.get("original_max_position_embeddings"))
    assert mod.rope_type == kind and mod.rotary_dim == rot
    assert torch.equal(mod.cos_cache, cos) and torch.equal(mod.sin_cache, sin)
    assert mod.operator_type == OperatorType.ROTARYEMBEDDING and mod.backend is None
    assert "rope_type=" in mod.extra_repr()


def test_unknown_kind_asserts_like_the_reference():
    with pytest.raises(AssertionError, match="Unsupported RoPE type"):
        RotaryEmbedding(dict(rope_type="yarn"), 64, 128, 10000.0)


def test_return_cos_sin_and_row_selection():
    mod = RotaryEmbedding(None, 64, 128, 10000.0)
    x = torch.zeros(2, 3, 64, dtype=torch.bfloat16)
    pos = torch.tensor([[0, 1, 2], [100, 101, 127]])
    cos, sin = mod(x, pos, return_cos_sin=True)
    want_c, want_s = rope_ref.lookup(mod.cos_cache, mod.sin_cache, pos, torch.bfloat16)
    assert torch.equal(cos, want_c) and torch.equal(sin, want_s)
    lr = RotaryEmbedding(dict(rope_type="longrope", short_factor=SHORT, long_factor=LONG), 64, 256, 10000.0,
                         original_max_position_embeddings=64)
    for ids in (torch.tensor([[1, 2, 3]]), torch.tensor([[63, 64, 65]])):
        assert torch.equal(lr.table_rows(ids), rope_ref.longrope_rows(ids, 64))
    off = torch.tensor([[2, 2, 2]])
    assert torch.equal(lr.table_rows(torch.tensor([[63, 64, 65]]), off), rope_ref.longrope_rows(torch.tensor([[63, 64, 65]]), 64, off))


def test_cpu_activations_are_refused():
    mod = RotaryEmbedding(None, 64, 128, 10000.0)
    x = torch.zeros(1, 2, 3, 64, dtype=torch.bfloat16)
    with pytest.raises(NotImplementedError, match="runs on the GPU"):
        mod(x, torch.tensor([[0, 1, 2]]))
    cos, sin = mod(x, torch.tensor([[0, 1, 2]]), return_cos_sin=True)
    with pytest.raises(NotImplementedError, match="device tensors"):
        mod.apply_rotary_emb(x, x, cos, sin)
