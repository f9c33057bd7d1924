"""Oracle: attention semantics of the reference, on CPU.

TEST INFRASTRUCTURE -- see ``oracle/__init__.py``.

Three restatements of ``softmax(Q K^T / sqrt(H) + M) V``:

* ``sdpa_native``        what the reference runs by default: torch's CPU
                         ``scaled_dot_product_attention`` on the tensors as given
                         (``pace/ops/backends/native.py:32-47``).
* ``sdpa_fp32``          the same library routine on fp32-upcast inputs: the
                         tolerance oracle for bf16 kernels that accumulate in fp32.
* ``sdpa_jit_emulated``  the oneDNN chain of ``torch.ops.pace.attention`` with its
                         intermediate tensor held in the input dtype
                         (``csrc/ops/kernels/attention_kernels.cpp:218-257``).
* ``sdpa_bruteforce_f64`` textbook loops in float64 for tiny inputs.

plus the op's argument checks (``csrc/ops/attention.cpp:26-87``) and the 4-D
causal mask the models pass down (``pace/llm/models/llama.py:284-310``).
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch
import torch.nn.functional as F

_FLOAT_TYPES = (torch.float32, torch.bfloat16)


def check_attention_args(q, k, v, mask, use_kq) -> int:
    """Argument checks of ``pace::attention`` in the reference's order.

    ``csrc/ops/attention.cpp:26-40`` (all 4-D, mask dereferenced so it is
    required), ``:42-50`` (K/V same shape), ``:52-67`` (dtypes), ``:77-87``
    (``use_KQ`` in {0, 1}).  Raises ``RuntimeError`` like ``TORCH_CHECK``.
    """
    if mask is None:
        raise RuntimeError("pace::SDPA attention requires 4D inputs, but recieved no attention mask")
    if not (q.dim() == 4 and k.dim() == 4 and v.dim() == 4 and mask.dim() == 4):
        raise RuntimeError(
            "pace::SDPA attention requires 4D inputs, but recieved: "
            f" input_Q - {list(q.shape)},  input_K - {list(k.shape)},  input_V - {list(v.shape)}, and "
            f" input_attention_mask - {list(mask.shape)}"
        )
    if k.shape != v.shape:
        raise RuntimeError(
            "pace::SDPA attention requires Key and Value sizes to be of same shape, but recieved: "
            f" input_K - {list(k.shape)},  input_V - {list(v.shape)}"
        )
    for name, t in (("Query", q), ("Key", k), ("Value", v), ("Attention mask", mask)):
        if t.dtype not in _FLOAT_TYPES:
            raise RuntimeError(
                f"pace::SDPA attention only support the dtypes Float and BF16 types for input {name}"
            )
    kq = 0 if use_kq is None else int(use_kq)
    if kq not in (0, 1):
        raise RuntimeError(f"pace::SDPA attention requires use_KQ to be 0 or 1 but recieved:  use_KQ - {kq}")
    return kq


def sdpa_native(q, k, v, mask=None):
    """``pace/ops/backends/native.py:44-47`` on CPU tensors."""
    return F.scaled_dot_product_attention(q, k, v, attn_mask=mask)


def sdpa_fp32(q, k, v, mask=None):
    """Library SDPA with everything upcast to fp32; result stays fp32."""
    m = None if mask is None else mask.float()
    return F.scaled_dot_product_attention(q.float(), k.float(), v.float(), attn_mask=m)


def sdpa_jit_emulated(q, k, v, mask=None):
    """Method 1 of ``attention_kernels.cpp:218-257``.

    ``S`` is a tensor of the *input* dtype (``dta``, ``:171,223-224``): the
    scaled product, the mask add and the softmax each round to that dtype
    before the next primitive reads it; every primitive accumulates in fp32.
    """
    dt = q.dtype
    scale = 1.0 / math.sqrt(q.shape[-1])  # :188
    s = (torch.matmul(q.float(), k.float().transpose(-1, -2)) * scale).to(dt)  # :229-237
    if mask is not None and mask.numel():
        s = (s.float() + mask.float()).to(dt)  # :240-242
    p = torch.softmax(s.float(), dim=-1).to(dt)  # :245
    return torch.matmul(p.float(), v.float()).to(dt)  # :248-255


def sdpa_bruteforce_f64(q, k, v, mask=None) -> np.ndarray:
    """Scalar-loop definition in float64; only for tiny shapes."""
    qn = q.double().numpy()
    kn = k.double().numpy()
    vn = v.double().numpy()
    B, N, S, H = qn.shape
    L = kn.shape[2]
    mn = None
    if mask is not None:
        mn = np.broadcast_to(mask.double().numpy(), (B, N, S, L))
    out = np.zeros((B, N, S, vn.shape[3]))
    for b in range(B):
        for n in range(N):
            for s in range(S):
                logits = np.empty(L)
                for t in range(L):
                    acc = 0.0
                    for h in range(H):
                        acc += qn[b, n, s, h] * kn[b, n, t, h]
                    logits[t] = acc / math.sqrt(H) + (mn[b, n, s, t] if mn is not None else 0.0)
                logits -= logits.max()
                w = np.exp(logits)
                w /= w.sum()
                for t in range(L):
                    out[b, n, s] += w[t] * vn[b, n, t]
    return out


def causal_mask_4d(
    attention_mask_2d: torch.Tensor, q_len: int, kv_len: int, dtype: torch.dtype
) -> torch.Tensor:
    """Additive ``[B, 1, q_len, kv_len]`` mask of ``llama.py:292-299``.

    The reference calls ``AttentionMaskConverter(is_causal=True).to_4d`` of
    transformers 4.51.3.  Closed form: entry ``(b, 0, s, t)`` is ``0`` when
    ``t <= (kv_len - q_len) + s`` and ``attention_mask_2d[b, t] == 1``, else
    ``finfo(dtype).min``.
    """
    past = kv_len - q_len
    t = torch.arange(kv_len).view(1, 1, 1, kv_len)
    s = torch.arange(q_len).view(1, 1, q_len, 1)
    allowed = (t <= past + s) & (attention_mask_2d[:, None, None, :kv_len] != 0)
    out = torch.full(allowed.shape, torch.finfo(dtype).min, dtype=dtype)
    return out.masked_fill(allowed, 0.0)


def lengths_mask_4d(
    seq_lens, q_len: int, kv_cols: int, dtype: torch.dtype, kv_start: Optional[torch.Tensor] = None
) -> torch.Tensor:
    """Mask equivalent to per-sequence lengths: row ``s`` of sequence ``b`` may read
    tokens ``kv_start[b] <= t <= seq_lens[b] - q_len + s``; everything else
    (including columns past the sequence) is ``finfo.min``.  This is the mask a
    right-padded ragged batch would get from ``causal_mask_4d`` + BMC padding
    (``cache.py:195-222``)."""
    lens = torch.as_tensor(seq_lens, dtype=torch.long).view(-1, 1, 1, 1)
    t = torch.arange(kv_cols).view(1, 1, 1, kv_cols)
    s = torch.arange(q_len).view(1, 1, q_len, 1)
    allowed = t <= (lens - q_len + s)
    if kv_start is not None:
        allowed &= t >= torch.as_tensor(kv_start, dtype=torch.long).view(-1, 1, 1, 1)
    out = torch.full(allowed.shape, torch.finfo(dtype).min, dtype=dtype)
    return out.masked_fill(allowed, 0.0)
