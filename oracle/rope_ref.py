"""Rotary position embedding of the reference, restated on the CPU.  TEST INFRASTRUCTURE ONLY.

Follows ``pace/ops/rotary_embedding.py``:

  * tables  -- ``cos_sin_tables`` restates the five table builders
               (``:62-199``) and the selection in ``RotaryEmbedding.__init__``
               (``:286-364``): rows are positions, columns the rotary_dim/2
               frequencies, values fp32.
  * lookup  -- ``lookup`` restates ``forward`` (``:370-410``): rows are picked
               by position id and converted to the dtype of the activations
               (so bf16 activations see bf16-rounded cos / sin).
  * rotate  -- ``rotate`` restates ``_apply_rotary_emb`` (``:412-443``) with the
               same sequence of tensor operations in the activations' dtype,
               which fixes the intermediate roundings for bf16:
                 o1 = rnd(rnd(x1*cos) - rnd(x2*sin)),  o2 = rnd(rnd(x2*cos) + rnd(x1*sin)).
               neox style pairs dim i with i + rot/2, GPT-J style 2i with 2i+1.

Pinning: the reference holds no test of this operator, so the restatement is
pinned by mathematics and by library routines (``tests/test_oracle_rope.py``):
complex multiplication by e^{i p w} in float64, norm preservation, position 0
is the identity, q_m . k_n depends on m - n only, an independent
round-to-nearest-even emulation of the bf16 steps written with integer bit
operations, and for the scaled tables the inverse frequencies of the installed
``transformers.modeling_rope_utils`` (``linear``, ``dynamic``, ``llama3``,
``longrope``).  The ``longrope`` *row selection* of ``forward`` (offset by the
original context length once any position exceeds it) picks the factors that
transformers' rule (``max id + 1`` exceeds the original length) picks, except
for a batch whose largest id equals the original length; that single point
follows the reference as written and is **parity unpinned**.
"""
from __future__ import annotations

import math
from typing import Any, Dict, Optional, Sequence, Tuple

import torch


def inv_freq(base: float, rotary_dim: int, rescale: Optional[Sequence[float]] = None) -> torch.Tensor:
    """``1 / (rescale * base^(2i/rot))`` -- ``rotary_embedding.py:62-84``."""
    expo = torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim
    f = base ** expo
    if rescale:
        f = torch.tensor(list(rescale), dtype=torch.float32) * f
    return 1.0 / f


def _tables_from(freq: torch.Tensor, rows: int, amplitude: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Outer product positions x frequencies, then cos / sin -- ``:87-103``."""
    ang = torch.outer(torch.arange(rows, dtype=torch.float), freq)
    return ang.cos() * amplitude, ang.sin() * amplitude


def llama3_freq(base: float, rotary_dim: int, factor: float, low: float, high: float, original_max: int) -> torch.Tensor:
    """Wavelength-dependent rescaling of the llama-3 family -- ``:151-186``."""
    f = inv_freq(base, rotary_dim)
    wavelen = 2 * math.pi / f
    low_wavelen = original_max / low
    high_wavelen = original_max / high
    smooth = (original_max / wavelen - low) / (high - low) if low != high else 0
    mid = (1 - smooth) * f / factor + smooth * f
    return torch.where(wavelen < high_wavelen, f, torch.where(wavelen > low_wavelen, f / factor, mid))


def cos_sin_tables(
    rope_scaling: Optional[Dict[str, Any]],
    rotary_dim: int,
    max_position_embeddings: int,
    rope_theta: float,
    partial_rotary_factor: float = 1.0,
    original_max_position_embeddings: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, str, int]:
    """(cos, sin, rope_type, rotary_dim) as ``RotaryEmbedding.__init__`` builds them (``:257-368``)."""
    if partial_rotary_factor < 1.0:
        rotary_dim = int(rotary_dim * partial_rotary_factor)
    kind = "default" if rope_scaling is None else rope_scaling.get("rope_type", rope_scaling.get("type"))
    if kind == "default":
        cos, sin = _tables_from(inv_freq(rope_theta, rotary_dim), max_position_embeddings)
    elif kind == "linear":
        # the reference scales the *amplitude* of cos / sin by the factor (``:119-130``, ``:100-101``)
        cos, sin = _tables_from(inv_freq(rope_theta, rotary_dim), max_position_embeddings, rope_scaling["scaling_factor"])
    elif kind == "dynamic":
        s = rope_scaling["scaling_factor"]
        rows = max_position_embeddings * s
        base = rope_theta * ((s * rows / max_position_embeddings) - (s - 1)) ** (rotary_dim / (rotary_dim - 2))
        cos, sin = _tables_from(inv_freq(base, rotary_dim), rows)
    elif kind == "llama3":
        f = llama3_freq(rope_theta, rotary_dim, rope_scaling["factor"], rope_scaling["low_freq_factor"],
                        rope_scaling["high_freq_factor"], rope_scaling["original_max_position_embeddings"])
        cos, sin = _tables_from(f, max_position_embeddings)
    elif kind == "longrope":
        orig = original_max_position_embeddings or max_position_embeddings
        ratio = max_position_embeddings / orig
        amp = 1.0 if ratio <= 1.0 else math.sqrt(1 + math.log(ratio) / math.log(orig))
        if rope_scaling.get("attention_factor") is not None:
            amp = rope_scaling["attention_factor"]
        cs, ss = _tables_from(inv_freq(rope_theta, rotary_dim, rope_scaling["short_factor"]), orig, amp)
        cl, sl = _tables_from(inv_freq(rope_theta, rotary_dim, rope_scaling["long_factor"]), max_position_embeddings, amp)
        cos, sin = torch.cat([cs, cl]), torch.cat([ss, sl])
    else:
        raise AssertionError(f"Unsupported RoPE type: {kind}")
    return cos, sin, kind, rotary_dim


def longrope_rows(position_ids: torch.Tensor, original_max: int, offsets: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Table rows the longrope variant reads (``:381-392``): every id is shifted by the
    original context length as soon as ANY id of the call exceeds it."""
    shift = (torch.any(position_ids > original_max).float() * torch.full_like(position_ids, original_max)).long()
    idx = position_ids + shift
    return idx + offsets if offsets is not None else idx


def lookup(cos: torch.Tensor, sin: torch.Tensor, rows: torch.Tensor, dtype: torch.dtype) -> Tuple[torch.Tensor, torch.Tensor]:
    """cos / sin rows for ``rows`` ([B, S] ids), converted to the activations' dtype (``:396-400``)."""
    flat = rows.flatten()
    c = cos.index_select(0, flat).unflatten(0, rows.shape).to(dtype)
    s = sin.index_select(0, flat).unflatten(0, rows.shape).to(dtype)
    return c, s


def rotate(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, neox: bool = True, rotary_dim: Optional[int] = None) -> torch.Tensor:
    """Rotate ``x`` [B, H, S, D] by cos / sin [B, S, rot/2] (already in ``x.dtype``).

    Dims beyond ``rotary_dim`` pass through (the longrope branch of the
    reference, ``:421-430``, and the slicing GPT-J does around the call,
    ``pace/llm/models/gptj.py:115-131``).  Operation order as ``:432-443``.
    """
    rot = x.shape[-1] if rotary_dim is None else rotary_dim
    c, s = cos.unsqueeze(1), sin.unsqueeze(1)
    xr, xp = x[..., :rot], x[..., rot:]
    if neox:
        x1, x2 = xr[..., : rot // 2], xr[..., rot // 2:]
    else:
        x1, x2 = xr[..., ::2], xr[..., 1::2]
    o1 = x1 * c - x2 * s
    o2 = x2 * c + x1 * s
    out = torch.cat((o1, o2), dim=-1) if neox else torch.stack((o1, o2), dim=-1).flatten(-2)
    return torch.cat((out, xp), dim=-1) if xp.shape[-1] else out


def rotate_longrope_form(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, rotary_dim: int) -> torch.Tensor:
    """The longrope branch as the reference writes it (``:421-430``): cos / sin repeated to
    rotary_dim columns and ``x*cos + rotate_half(x)*sin``.  Same values as ``rotate(neox)``:
    negation is exact and commutes with rounding."""
    c = cos.unsqueeze(1).repeat(1, 1, 1, 2)
    s = sin.unsqueeze(1).repeat(1, 1, 1, 2)
    xr, xp = x[..., :rotary_dim], x[..., rotary_dim:]
    half = torch.cat((-xr[..., rotary_dim // 2:], xr[..., : rotary_dim // 2]), dim=-1)
    return torch.cat((xr * c + half * s, xp), dim=-1)


def rope_then_append_reference(q, k, v, cos, sin, neox=True):
    """The step the models run before the cache (``pace/llm/models/llama.py:147-158``):
    rotate q and k, leave v; returns what is handed to ``update_cache`` and to attention."""
    return rotate(q, cos, sin, neox), rotate(k, cos, sin, neox), v
