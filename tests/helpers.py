"""Seeded input builders shared by the parity tests."""
from __future__ import annotations

import numpy as np
import torch


def seeded_kv(seed, batch, heads, tokens, dim, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(batch, heads, tokens, dim, generator=g).to(dtype)
    v = torch.randn(batch, heads, tokens, dim, generator=g).to(dtype)
    return k, v


def seeded_q(seed, batch, heads, q_len, dim, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(batch, heads, q_len, dim, generator=g).to(dtype)


def assert_bits_equal(a: torch.Tensor, b: torch.Tensor, what: str = "") -> None:
    a = a.detach().cpu().contiguous()
    b = b.detach().cpu().contiguous()
    assert a.shape == b.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(b.shape)}"
    assert a.dtype == b.dtype, f"{what}: dtype {a.dtype} vs {b.dtype}"
    same = torch.equal(a.view(torch.int16) if a.dtype == torch.bfloat16 else a, b.view(torch.int16) if b.dtype == torch.bfloat16 else b)
    if not same:
        diff = (a.float() != b.float()).nonzero()
        raise AssertionError(f"{what}: {diff.shape[0]} elements differ, first at {diff[0].tolist()}")


# Attention tolerance of the hot path: bf16 inputs/outputs, fp32 accumulation.
ATTN_ATOL = 2e-2
ATTN_RTOL = 1e-2


def assert_attention_close(out: torch.Tensor, ref_fp32: torch.Tensor, what: str = "") -> None:
    o = out.detach().float().cpu()
    r = ref_fp32.detach().float().cpu()
    assert o.shape == r.shape, f"{what}: shape {tuple(o.shape)} vs {tuple(r.shape)}"
    err = (o - r).abs()
    bound = ATTN_ATOL + ATTN_RTOL * r.abs()
    bad = err > bound
    assert not torch.isnan(o).any(), f"{what}: NaN in output"
    if bad.any():
        idx = bad.nonzero()[0].tolist()
        raise AssertionError(
            f"{what}: {int(bad.sum())} of {bad.numel()} outside atol={ATTN_ATOL} rtol={ATTN_RTOL}; "
            f"max abs err {err.max().item():.4g} at first bad index {idx}: got {o[tuple(idx)].item():.5g} want {r[tuple(idx)].item():.5g}"
        )
