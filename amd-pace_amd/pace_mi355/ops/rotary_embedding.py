"""Rotary position embedding operator with the reference's interface
(``pace/ops/rotary_embedding.py:202-481``), executed by the gfx950 library.

The constructor builds the same ``cos_cache`` / ``sin_cache`` buffers
(rows = positions, columns = rotary_dim / 2 frequencies) for the reference's five
scaling kinds.  ``forward`` returns a callable, as the reference does, but one that
keeps the *table rows* of the tokens instead of gathered cos / sin tensors, so the
rotation can run

  * on dense tensors            -- ``rope(query=q, key=k)``            -> ``pace_rope_apply``
  * folded into the cache append -- ``cache.update_cache(k, v, 2, rope=rope)``
                                                                     -> ``pace_rope_append_paged``
  * folded into the attention launch together with the append (decode / verify steps).

Device tensors only (there is no second implementation): bf16 with head_dim 64, 96, 128 or 256 and
a rotary_dim that is a multiple of 16, or fp32 with any even head_dim / rotary_dim (dense form only);
``[B, H, S, D]`` (``unsqueeze_dim=1``) or ``[B, S, H, D]`` (``unsqueeze_dim=2``).
"""
from __future__ import annotations

import ctypes
import math
from typing import Any, Callable, Dict, Optional, Tuple, Union

import torch

from .. import _native as nat
from ..utils.logging import PACE_ASSERT
from .base import OperatorBase
from .enum import BackendType, OperatorType


def _frequencies(base: float, rotary_dim: int, rescale=None) -> torch.Tensor:
    expo = torch.arange(0, rotary_dim, 2, dtype=torch.float) / rotary_dim
    scale = torch.tensor(rescale, dtype=torch.float32) if rescale else 1
    return 1.0 / (scale * (base ** expo))


def _table(freq: torch.Tensor, rows, amplitude: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    angles = torch.einsum("i,j -> ij", torch.arange(rows, dtype=torch.float), freq)
    return angles.cos() * amplitude, angles.sin() * amplitude


def _default_tables(cfg, dim, rows, theta, **_):
    return _table(_frequencies(theta, dim), rows)


def _linear_tables(cfg, dim, rows, theta, **_):
    # the factor multiplies cos / sin themselves, as in the reference (:119-130)
    return _table(_frequencies(theta, dim), rows, cfg["scaling_factor"])


def _dynamic_tables(cfg, dim, rows, theta, **_):
    s = cfg["scaling_factor"]
    longest = rows * s
    theta = theta * ((s * longest / rows) - (s - 1)) ** (dim / (dim - 2))
    return _table(_frequencies(theta, dim), longest)


def _llama3_tables(cfg, dim, rows, theta, **_):
    f = _frequencies(theta, dim)
    factor, low, high = cfg["factor"], cfg["low_freq_factor"], cfg["high_freq_factor"]
    orig = cfg["original_max_position_embeddings"]
    wavelen = 2 * math.pi / f
    smooth = (orig / wavelen - low) / (high - low) if low != high else 0
    f = torch.where(
        wavelen < orig / high,
        f,
        torch.where(wavelen > orig / low, f / factor, (1 - smooth) * f / factor + smooth * f),
    )
    return _table(f, rows)


_TABLE_BUILDERS: Dict[str, Callable] = {
    "default": _default_tables,
    "linear": _linear_tables,
    "dynamic": _dynamic_tables,
    "llama3": _llama3_tables,
}


def _check_rows(x: torch.Tensor, name: str) -> None:
    if not x.is_cuda or x.dtype not in (torch.bfloat16, torch.float32) or x.dim() != 4:
        raise NotImplementedError(f"rotary embedding runs on bf16 / fp32 device tensors of four dims; {name} is "
                                  f"{x.dtype} {tuple(x.shape)} on {x.device}")
    if x.dtype == torch.bfloat16 and x.shape[-1] not in (64, 96, 128, 256):
        raise NotImplementedError(f"rotary embedding on bf16 supports head_dim 64, 96, 128 or 256, got {x.shape[-1]}")
    if x.shape[-1] % 2:
        raise NotImplementedError(f"rotary embedding needs an even head_dim, got {x.shape[-1]}")


def _strided(x: torch.Tensor) -> torch.Tensor:
    step = 8 if x.dtype == torch.bfloat16 else 1  # bf16 rows move in 16-byte chunks
    ok = x.stride(3) == 1 and x.data_ptr() % 16 == 0 and all(
        s % step == 0 and (s > 0 or n == 1) for s, n in zip(x.stride()[:3], x.shape[:3]))
    return x if ok else x.contiguous()


def launch_rope_apply(desc: nat.RopeDesc, query: Optional[torch.Tensor], key: Optional[torch.Tensor],
                      unsqueeze_dim: int = 1, rows_shape: Optional[Tuple[int, int]] = None):
    """Rotate dense ``query`` / ``key`` into new tensors with ``pace_rope_apply`` (bf16) or
    ``pace_rope_apply_f32``.  ``unsqueeze_dim`` names the head axis as the reference does
    (``pace/ops/rotary_embedding.py:418-419``): 1 for ``[B, H, S, D]``, 2 for ``[B, S, H, D]``.
    ``rows_shape``: shape of the position rows behind ``desc``; ``(1, S)`` rows serve every sequence,
    as the reference's broadcast of ``cos.unsqueeze(1)`` does."""
    if unsqueeze_dim not in (1, 2):
        raise NotImplementedError(f"rotary embedding takes [B, H, S, D] (unsqueeze_dim=1) or [B, S, H, D] (2), not {unsqueeze_dim}")
    t_ax, h_ax = (2, 1) if unsqueeze_dim == 1 else (1, 2)
    outs = []
    args = []
    ref = query if query is not None else key
    B, S, D = ref.shape[0], ref.shape[t_ax], ref.shape[3]
    if rows_shape is not None:
        if tuple(rows_shape) not in ((B, S), (1, S)):
            raise RuntimeError(f"position rows {tuple(rows_shape)} fit neither [B={B}, S={S}] nor [1, S={S}]")
        if rows_shape[0] == 1:
            desc.pos_stride_b = 0
    for x, name in ((query, "query"), (key, "key")):
        if x is None:
            outs.append(None)
            args += [None, None, 0, 0, 0, 0]
            continue
        _check_rows(x, name)
        if x.shape[0] != B or x.shape[t_ax] != S or x.shape[3] != D or x.dtype != ref.dtype:
            raise RuntimeError(f"query / key disagree: {tuple(query.shape)} {query.dtype} vs {tuple(key.shape)} {key.dtype}")
        xin = _strided(x)
        out = torch.empty_strided(xin.shape, xin.stride(), dtype=xin.dtype, device=xin.device) if xin is x else xin
        outs.append(out)
        args += [xin.data_ptr(), out.data_ptr(), xin.stride(0), xin.stride(h_ax), xin.stride(t_ax), xin.shape[h_ax]]
    fn = nat.load().pace_rope_apply if ref.dtype == torch.bfloat16 else nat.load().pace_rope_apply_f32
    nat.check(fn(ctypes.byref(desc), *args, B, S, D, nat.current_stream_ptr()))
    return outs[0], outs[1]


class RopeCall:
    """What ``RotaryEmbedding.forward`` returns: the rotation of one model step.

    Callable like the reference's ``partial(apply_rotary_emb, cos=..., sin=...)``:
    ``rope(query=q, key=k)`` or ``rope(q, k, is_neox_style=False)``.  The cache and
    the attention backend take the object itself to fold the rotation into their launches.
    """

    def __init__(self, module: "RotaryEmbedding", rows: torch.Tensor):
        self.module = module
        self.rows = rows  # int32 [B, S] (or [1, S]) table rows, on the device
        self.is_neox_style = True

    def desc(self, is_neox_style: Optional[bool] = None, dtype: torch.dtype = torch.bfloat16) -> nat.RopeDesc:
        neox = self.is_neox_style if is_neox_style is None else is_neox_style
        if self.module.rope_type == "longrope":
            neox = True  # the reference's longrope branch always pairs dim i with i + rotary_dim / 2 (:421-430)
        cos, sin = self.module.device_tables(self.rows.device, dtype)
        d = nat.RopeDesc()
        d.cos, d.sin = cos.data_ptr(), sin.data_ptr()
        d.table_dtype = nat.DTYPE_BF16 if dtype == torch.bfloat16 else nat.DTYPE_F32
        d.table_rows, d.rotary_dim = cos.shape[0], 2 * cos.shape[1]
        d.interleaved = 0 if neox else 1
        d.positions = self.rows.data_ptr()
        d.pos_stride_b = 0 if self.rows.shape[0] == 1 else self.rows.stride(0)
        return d

    def with_style(self, is_neox_style: bool) -> "RopeCall":
        other = RopeCall(self.module, self.rows)
        other.is_neox_style = bool(is_neox_style)
        return other

    def __call__(self, query: torch.Tensor, key: torch.Tensor, is_neox_style: Optional[bool] = None, unsqueeze_dim: int = 1):
        ref = query if query is not None else key
        return launch_rope_apply(self.desc(is_neox_style, ref.dtype), query, key, unsqueeze_dim, tuple(self.rows.shape))


class RotaryEmbedding(OperatorBase):
    """Reference signature (``pace/ops/rotary_embedding.py:257-268``)."""

    @property
    def operator_type(self) -> OperatorType:
        return OperatorType.ROTARYEMBEDDING

    def __init__(
        self,
        rope_scaling: Optional[Dict[str, Any]],
        rotary_dim: int,
        max_position_embeddings: int,
        rope_theta: Union[int, float],
        partial_rotary_factor: float = 1.0,
        dtype: Optional[torch.dtype] = None,
        backend_impl: Optional[BackendType] = None,  # unused, as in the reference
        **rope_kwargs,
    ):
        super().__init__(backend_impl=backend_impl, dtype=dtype)
        if partial_rotary_factor < 1.0:
            rotary_dim = int(rotary_dim * partial_rotary_factor)
        self.rotary_dim = rotary_dim
        self.partial_rotary_factor = partial_rotary_factor
        self.rope_kwargs = rope_kwargs
        self.rope_scaling = rope_scaling
        self.rope_type = "default" if rope_scaling is None else rope_scaling.get("rope_type", rope_scaling.get("type"))
        self.max_position_embeddings = max_position_embeddings
        self.rope_theta = rope_theta
        if self.rope_type == "longrope":
            cos, sin = self._longrope_tables()
        else:
            PACE_ASSERT(self.rope_type in _TABLE_BUILDERS, f"Unsupported RoPE type: {self.rope_type}")
            cos, sin = _TABLE_BUILDERS[self.rope_type](rope_scaling, rotary_dim, max_position_embeddings, rope_theta)
        self.register_buffer("cos_cache", cos, persistent=False)
        self.register_buffer("sin_cache", sin, persistent=False)
        self._device_tables: Dict[Any, Tuple[torch.Tensor, torch.Tensor]] = {}

    def _longrope_tables(self):
        cfg, rows = self.rope_scaling, self.max_position_embeddings
        orig = self.rope_kwargs.get("original_max_position_embeddings", rows)
        self.original_max_position_embeddings = orig
        ratio = rows / orig
        amp = 1.0 if ratio <= 1.0 else math.sqrt(1 + math.log(ratio) / math.log(orig))
        if cfg.get("attention_factor") is not None:
            amp = cfg["attention_factor"]
        short = _table(_frequencies(self.rope_theta, self.rotary_dim, cfg["short_factor"]), orig, amp)
        long_ = _table(_frequencies(self.rope_theta, self.rotary_dim, cfg["long_factor"]), rows, amp)
        return torch.cat([short[0], long_[0]], dim=0), torch.cat([short[1], long_[1]], dim=0)

    def device_tables(self, device, dtype: torch.dtype = torch.bfloat16) -> Tuple[torch.Tensor, torch.Tensor]:
        """Copies of the tables on ``device`` in the activations' dtype (the reference's ``.to(x.dtype)``, ``:398-399``)."""
        key = (str(device), dtype)
        if key not in self._device_tables:
            self._device_tables[key] = (
                self.cos_cache.to(device=device, dtype=dtype).contiguous(),
                self.sin_cache.to(device=device, dtype=dtype).contiguous(),
            )
        return self._device_tables[key]

    def table_rows(self, position_ids: torch.Tensor, offsets: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Rows of the tables the tokens read (reference ``forward``, ``:381-394``)."""
        if self.rope_type == "longrope":
            k = self.original_max_position_embeddings
            shift = (torch.any(position_ids > k).float() * torch.full_like(position_ids, k)).long()
            idx = position_ids + shift
            return idx + offsets if offsets is not None else idx
        return position_ids

    def forward(self, x: torch.Tensor, position_ids: torch.Tensor, return_cos_sin: bool = False,
                offsets: Optional[torch.Tensor] = None):
        rows = self.table_rows(position_ids, offsets)
        if return_cos_sin:
            flat = rows.flatten().to(self.cos_cache.device)
            cos = self.cos_cache.index_select(0, flat).unflatten(0, rows.shape).to(x.dtype)
            sin = self.sin_cache.index_select(0, flat).unflatten(0, rows.shape).to(x.dtype)
            return cos, sin
        if not x.is_cuda:
            raise NotImplementedError("rotary embedding runs on the GPU; activations are on " + str(x.device))
        return RopeCall(self, rows.to(device=x.device, dtype=torch.int32).contiguous())

    def apply_rotary_emb(self, query: torch.Tensor, key: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                         unsqueeze_dim: int = 1, is_neox_style: bool = True):
        """Rotate with gathered ``cos`` / ``sin`` ``[B | 1, S, rotary_dim/2]`` (reference ``:445-474``)."""
        ref = query if query is not None else key
        _check_rows(ref, "query")
        if cos.dim() != 3 or sin.shape != cos.shape:
            raise RuntimeError(f"cos / sin must be [B, S, rotary_dim/2]; got {tuple(cos.shape)} and {tuple(sin.shape)}")
        nb, S = cos.shape[0], cos.shape[1]
        cos2 = cos.to(device=ref.device, dtype=ref.dtype).reshape(nb * S, -1).contiguous()
        sin2 = sin.to(device=ref.device, dtype=ref.dtype).reshape(nb * S, -1).contiguous()
        rows = torch.arange(nb * S, dtype=torch.int32, device=ref.device).view(nb, S)
        d = nat.RopeDesc()
        d.cos, d.sin = cos2.data_ptr(), sin2.data_ptr()
        d.table_dtype = nat.DTYPE_BF16 if ref.dtype == torch.bfloat16 else nat.DTYPE_F32
        d.table_rows, d.rotary_dim = nb * S, 2 * cos2.shape[1]
        d.interleaved = 0 if (is_neox_style or self.rope_type == "longrope") else 1  # longrope: always halves (:421-430)
        d.positions, d.pos_stride_b = rows.data_ptr(), rows.stride(0)
        return launch_rope_apply(d, query, key, unsqueeze_dim, (nb, S))

    def extra_repr(self) -> str:
        return (f"rope_type={self.rope_type}, rotary_dim={self.rotary_dim}, "
                f"max_position_embeddings={self.max_position_embeddings}, rope_theta={self.rope_theta}")
