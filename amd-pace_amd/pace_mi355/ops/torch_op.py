"""``torch.ops.pace.attention`` with the reference's schema and argument checks.

Schema string copied from the interface the reference registers
(``csrc/ops/attention.cpp:104-108``); checks and their order follow
``csrc/ops/attention.cpp:26-87``: 4-D inputs, K/V same shape, dtypes, ``use_KQ``.
The computation is ``pace_attn_dense`` of the HIP library; the op has no CPU
implementation.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _native as nat

_SCHEMA = "attention(Tensor input_Q, Tensor input_K, Tensor input_V, Tensor ? input_mask, Scalar ? use_KQ) -> Tensor"
_FLOATS = (torch.float32, torch.bfloat16)

_lib = torch.library.Library("pace", "FRAGMENT")
_lib.define(_SCHEMA)


def _check(q, k, v, mask, use_kq) -> None:
    if mask is None:
        raise RuntimeError("pace::SDPA attention requires 4D inputs, but recieved no input_attention_mask")
    if not (q.dim() == 4 and k.dim() == 4 and v.dim() == 4 and mask.dim() == 4):
        raise RuntimeError(
            "pace::SDPA attention requires 4D inputs, but recieved:  input_Q - "
            f"{list(q.shape)},  input_K - {list(k.shape)},  input_V - {list(v.shape)}, and  input_attention_mask - {list(mask.shape)}"
        )
    if k.shape != v.shape:
        raise RuntimeError(
            "pace::SDPA attention requires Key and Value sizes to be of same shape, but recieved:  input_K - "
            f"{list(k.shape)},  input_V - {list(v.shape)}"
        )
    for what, t in (("Query", q), ("Key", k), ("Value", v), ("Attention mask", mask)):
        if t.dtype not in _FLOATS:
            raise RuntimeError(f"pace::SDPA attention only support the dtypes Float and BF16 types for input {what}")
    kq = 0 if use_kq is None else int(use_kq)
    if kq not in (0, 1):
        raise RuntimeError(f"pace::SDPA attention requires use_KQ to be 0 or 1 but recieved:  use_KQ - {kq}")


def _attention(input_Q, input_K, input_V, input_mask: Optional[torch.Tensor] = None, use_KQ=None):
    _check(input_Q, input_K, input_V, input_mask, use_KQ)
    q, k, v, m = input_Q, input_K, input_V, input_mask
    if not q.is_cuda:
        raise RuntimeError("pace::attention of this package runs on the GPU only; move the tensors to the device")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError("pace::SDPA attention only support the dtypes Float and BF16 types for input Query/Key/Value of one dtype")
    B, N, S, H = q.shape
    L = k.shape[2]
    if k.shape[0] != B or k.shape[1] != N or k.shape[3] != H:
        raise RuntimeError(f"pace::SDPA attention: Key {list(k.shape)} does not match Query {list(q.shape)}")
    if m.shape[3] != L:
        raise RuntimeError(f"pace::SDPA attention: mask {list(m.shape)} does not match key length {L}")
    # The reference reads its operands as dense row-major buffers
    # (csrc/pace_tensor/pace_aten_interface.cpp:151-179).
    q, k, v, m = q.contiguous(), k.contiguous(), v.contiguous(), m.contiguous()
    out = torch.empty(q.shape, dtype=q.dtype, device=q.device)
    dt = nat.DTYPE_F32 if q.dtype == torch.float32 else nat.DTYPE_BF16
    mdt = nat.DTYPE_F32 if m.dtype == torch.float32 else nat.DTYPE_BF16
    lib = nat.load()
    # scratch for the library's look over the mask (prefill-sized bf16 calls; 0 bytes otherwise)
    ws_bytes = int(lib.pace_attn_dense_workspace_bytes(dt, S, H, 1, m.shape[0], m.shape[1], m.shape[2]))
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes else None
    nat.check(
        lib.pace_attn_dense_ws(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), out.data_ptr(), dt, B, N, S, L, H,
            m.data_ptr(), mdt, m.shape[0], m.shape[1], m.shape[2],
            ws.data_ptr() if ws is not None else None, ws_bytes, nat.current_stream_ptr(),
        )
    )
    return out


_lib.impl("attention", _attention, "CompositeExplicitAutograd")
