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


# Attention tolerance of the hot path (bf16 inputs / outputs, fp32 accumulation), two caps that both hold:
# the largest absolute error of any output element, and the relative error of the compared output
# (Euclidean norm of the error over the norm of the fp32 oracle's output).
ATTN_MAX_ABS = 2e-2
ATTN_MAX_REL = 1e-2

# (test id, label, max abs error, relative error, elements) of every comparison made in this process;
# conftest.py prints the worst per test at the end of the run.
OBSERVED = []


def attention_errors(out: torch.Tensor, ref_fp32: torch.Tensor):
    """(max abs error, |out - ref|_2 / |ref|_2).  An oracle output that is all zeros has no relative error
    (0 is returned) and is held to the absolute cap alone."""
    o = out.detach().float().cpu()
    r = ref_fp32.detach().float().cpu()
    err = (o - r).abs()
    max_abs = float(err.max()) if err.numel() else 0.0
    e2, r2 = float(err.double().pow(2).sum().sqrt()), float(r.double().pow(2).sum().sqrt())
    return max_abs, (e2 / r2 if r2 > 0 else 0.0)


def assert_attention_close(out: torch.Tensor, ref_fp32: torch.Tensor, what: str = "") -> None:
    import os

    o = out.detach().float().cpu()
    r = ref_fp32.detach().float().cpu()
    assert o.shape == r.shape, f"{what}: shape {tuple(o.shape)} vs {tuple(r.shape)}"
    assert not torch.isnan(o).any(), f"{what}: NaN in output"
    max_abs, rel = attention_errors(o, r)
    test = os.environ.get("PYTEST_CURRENT_TEST", "").split(" ")[0]
    OBSERVED.append((test, what, max_abs, rel, o.numel()))
    print(f"[attention-error] {what}: max abs {max_abs:.3e} (cap {ATTN_MAX_ABS}), relative {rel:.3e} (cap {ATTN_MAX_REL}), "
          f"{o.numel()} elements")
    if max_abs > ATTN_MAX_ABS:
        err = (o - r).abs()
        idx = (err == err.max()).nonzero()[0].tolist()
        raise AssertionError(
            f"{what}: max abs err {max_abs:.4g} > {ATTN_MAX_ABS} at {idx}: got {o[tuple(idx)].item():.5g} want {r[tuple(idx)].item():.5g}; "
            f"{int((err > ATTN_MAX_ABS).sum())} of {err.numel()} elements over the cap")
    if rel > ATTN_MAX_REL:
        raise AssertionError(f"{what}: relative error {rel:.4g} > {ATTN_MAX_REL} (max abs err {max_abs:.4g})")
