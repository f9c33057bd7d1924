"""GPU parity: torch.ops.pace.attention (dense op of the reference) against the oracle."""
import numpy as np
import pytest
import torch

import pace_mi355.ops  # noqa: F401  (defines torch.ops.pace.attention)
from helpers import assert_attention_close, seeded_kv, seeded_q
from oracle.attention_ref import sdpa_fp32, sdpa_native

pytestmark = pytest.mark.gpu


def _mask(seed, shape, dtype):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)).to(dtype)


# Shapes drawn from the reference's property test (tests/ops/test_sdpa.py:83-91): B in {1,32,96},
# N in {1,16,32}, H in {1,64,128}, S in {1,128,512}, L in {1,512,2048}; sized to run in seconds.
CASES = [
    (1, 1, 1, 1, 1), (1, 16, 128, 64, 512), (32, 1, 1, 128, 2048), (2, 32, 512, 128, 1), (3, 2, 17, 1, 33),
    (2, 16, 1, 64, 2048), (96, 1, 1, 64, 1), (1, 1, 128, 128, 512), (2, 3, 5, 80, 70), (1, 2, 33, 256, 40),
    (2, 4, 1, 96, 700), (1, 3, 100, 96, 333), (2, 2, 1, 256, 900), (1, 2, 70, 256, 130), (1, 2, 9, 100, 50),
    # head sizes off every built one: not a multiple of 4 (element by element), 30 (the 32 build), 80 over several tiles
    (1, 2, 40, 50, 90), (1, 2, 20, 30, 45), (1, 2, 64, 80, 300),
    # the smallest build on the walk that shares its tiles (half a tile of chunks per load), exact and padded
    (1, 2, 48, 32, 100), (2, 1, 100, 28, 75),
]


# use_KQ selects an experimental path of the same function in the reference: two shapes suffice for it
@pytest.mark.parametrize("B,N,S,H,L,use_kq", [c + (False,) for c in CASES] + [CASES[1] + (True,), CASES[4] + (True,)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_dense_op_matches_oracle(device, B, N, S, H, L, dtype, use_kq):
    k, v = seeded_kv(1, B, N, L, H, dtype)
    q = seeded_q(2, B, N, S, H, dtype)
    m = _mask(3, (B, 1, 1, L), dtype)  # the reference test's mask: random additive bias of shape (B,1,1,L)
    out = torch.ops.pace.attention(q.to(device), k.to(device), v.to(device), m.to(device), use_kq)
    assert out.dtype == dtype and out.shape == q.shape and out.is_contiguous()
    ref = sdpa_fp32(q, k, v, m)
    if dtype == torch.float32:
        assert torch.allclose(out.cpu(), ref, atol=1e-5, rtol=1e-5), (out.cpu() - ref).abs().max()
    else:
        assert_attention_close(out, ref, "dense bf16")
        # and the reference's own bar: 1e-1 against torch's bf16 result (tests/ops/test_sdpa.py:113-127)
        assert torch.allclose(out.cpu().float(), sdpa_native(q, k, v, m).float(), atol=1e-1, rtol=1e-1)


@pytest.mark.parametrize("mshape", [(1, 1, 1, 40), (2, 1, 7, 40), (2, 3, 7, 40), (1, 3, 1, 40)])
def test_dense_op_mask_broadcast_and_mixed_dtypes(device, mshape):
    q, (k, v) = seeded_q(5, 2, 3, 7, 64), seeded_kv(6, 2, 3, 40, 64)
    m = _mask(7, mshape, torch.float32)  # fp32 mask with bf16 tensors
    out = torch.ops.pace.attention(q.to(device), k.to(device), v.to(device), m.to(device), 0)
    assert_attention_close(out, sdpa_fp32(q, k, v, m), f"mask {mshape}")


# Prefill-sized calls (more than 64 query rows) take the kernel whose waves share K / V through
# LDS: ragged row and key counts, every mask form it distinguishes, head counts off a multiple of 8.
@pytest.mark.parametrize("B,N,S,H,L,mask", [
    (1, 3, 200, 128, 333, "causal-bf16"),   # element-wise mask loads (L % 8 != 0), partial last unit
    (2, 5, 130, 128, 264, "causal-bf16"),   # 16-byte mask loads, L % 32 != 0
    (1, 8, 65, 64, 96, "causal-f32"),       # fp32 mask with bf16 tensors
    (2, 2, 512, 64, 512, "rows-bf16"),      # one mask line per batch entry
    (1, 40, 256, 128, 256, "causal-bf16"),  # enough workgroups for two tiles per wave
    (1, 9, 100, 128, 40, None),             # no mask (C ABI; the torch op always passes one)
    # 256 workgroups and more: two query tiles per wave
    (2, 32, 512, 128, 72, "causal-bf16"),
    (2, 32, 500, 64, 41, "causal-f32"),
    (2, 32, 512, 64, 104, "causal-bf16"),
    (2, 32, 512, 128, 50, None),
    (1, 33, 1000, 128, 96, "heads-bf16"),   # one mask plane per head; head count off a multiple of 8
    # rows masked everywhere with finfo.min (the first S - L rows of a causal mask with more rows than
    # keys; the pad rows of a left-padded batch look the same): the reference's softmax turns them into
    # the plain average of V, in every kernel the op can take
    (2, 32, 512, 128, 72, "causal-short-bf16"),
    (1, 4, 100, 64, 41, "causal-short-f32"),
    (2, 3, 20, 64, 8, "causal-short-bf16"),
    (1, 2, 40, 128, 70, "rows-masked-bf16"),
    # head_dim 256: rows of a head share K / V through LDS here too, one tile per wave, in every mask form
    (1, 3, 200, 256, 333, "causal-bf16"),
    (2, 4, 130, 256, 264, "causal-bf16"),
    (1, 2, 100, 256, 96, "causal-f32"),
    (1, 2, 100, 256, 50, None),
    (1, 5, 300, 256, 96, "heads-bf16"),
    (1, 2, 90, 256, 41, "causal-short-bf16"),
    (1, 2, 80, 256, 70, "rows-masked-bf16"),
    # head_dim 96 (a unit's chunks do not divide evenly over the workgroup's threads)
    (1, 3, 200, 96, 333, "causal-bf16"),
    (2, 32, 512, 96, 72, "causal-bf16"),
    (1, 2, 100, 96, 96, "causal-f32"),
    (2, 32, 300, 96, 50, None),
    (1, 2, 90, 96, 41, "causal-short-bf16"),
    # head sizes between 64 and 96 (OPT-2.7B's 80): the 96 build reading the rows as if padded with zeros
    (1, 3, 200, 80, 333, "causal-bf16"),
    (2, 4, 130, 72, 264, "causal-bf16"),
    (1, 2, 100, 88, 96, "causal-f32"),
    (2, 32, 300, 80, 50, None),
    (1, 2, 90, 80, 41, "causal-short-bf16"),
    (2, 3, 40, 80, 700, "rows-bf16"),          # few query rows: the kernel that splits the keys
    (2, 3, 1, 88, 333, "rows-bf16"),
])
def test_dense_prefill_shapes(device, B, N, S, H, L, mask):
    from oracle.attention_ref import causal_mask_4d
    from pace_mi355 import _native as nat

    k, v = seeded_kv(11, B, N, L, H)
    q = seeded_q(12, B, N, S, H)
    if mask is None:
        m = None
    elif mask.startswith("rows-masked"):  # every third row masked everywhere, long enough for several waves
        m = _mask(16, (B, 1, S, L), torch.bfloat16)
        m[:, :, ::3, :] = torch.finfo(torch.bfloat16).min
    elif mask.startswith("causal"):
        dt = torch.float32 if mask.endswith("f32") else torch.bfloat16
        if L >= S or "short" in mask:
            m = causal_mask_4d(torch.ones(B, L, dtype=torch.long), S, L, dt)
        else:  # more rows than keys: a banded finfo.min pattern that leaves every row something to read
            band = (torch.arange(L)[None, :] + torch.arange(S)[:, None]) % 3 == 0
            m = torch.zeros(B, 1, S, L, dtype=dt).masked_fill(band, torch.finfo(dt).min)
        m = m + _mask(13, (B, 1, S, L), dt) * (m == 0)  # a bias on the readable part as well
    elif mask.startswith("heads"):
        m = _mask(15, (B, N, S, L), torch.bfloat16)
    else:
        m = _mask(14, (B, 1, 1, L), torch.bfloat16)
    qd, kd, vd = q.to(device), k.to(device), v.to(device)
    if m is not None:
        out = torch.ops.pace.attention(qd, kd, vd, m.to(device), 0)
    else:
        out = torch.empty_like(qd)
        nat.check(nat.load().pace_attn_dense(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), out.data_ptr(), nat.DTYPE_BF16,
                                             B, N, S, L, H, None, nat.DTYPE_BF16, 1, 1, 1, nat.current_stream_ptr()))
    assert_attention_close(out, sdpa_fp32(q, k, v, m), f"prefill {B}x{N}x{S}x{H}x{L} {mask}")


@pytest.mark.parametrize("B,N,S,H,L,pad,mdt,mB", [
    (2, 32, 512, 128, 512, 0, torch.bfloat16, 2),     # the plain causal mask of a prompt
    (2, 32, 300, 128, 333, 45, torch.bfloat16, 2),    # left-padded by 45 columns, a partial last unit, rows before the keys' end
    (1, 40, 256, 64, 256, 0, torch.float32, 1),       # head_dim 64, fp32 mask, one mask for the whole batch
    (2, 32, 260, 64, 203, 32, torch.bfloat16, 2),     # padding that ends on a unit, a last row group that is partly filled
    (3, 16, 512, 128, 1100, 7, torch.bfloat16, 1),    # a chunk on top of a longer context (rows start at column 588)
])
def test_dense_prefill_with_plain_mask_lines(device, B, N, S, H, L, pad, mdt, mB):
    """Masks whose lines are 0 over one stretch of columns and finfo.min elsewhere (causal, with or without left
    padding): the op looks over the mask once and walks such rows by their first and last column, fetching K / V
    straight into LDS.  One sequence's lines are made unplain (a bias; a hole) so that both walks run in one call."""
    k, v = seeded_kv(31, B, N, L, H)
    q = seeded_q(32, B, N, S, H)
    past = L - S if L >= S else 0
    cols, rows = torch.arange(L)[None, :], torch.arange(S)[:, None]
    allowed = (cols <= rows + past) & (cols >= pad)
    m = torch.zeros(mB, 1, S, L, dtype=mdt).masked_fill(~allowed[None, None], torch.finfo(mdt).min)
    if mB > 1:
        m[1, :, : S // 2, pad] -= 0.5                      # finite and not 0: these lines are read
        m[1, :, S // 2 :, pad + 1] = torch.finfo(mdt).min  # a hole inside the stretch
    out = torch.ops.pace.attention(q.to(device), k.to(device), v.to(device), m.to(device), 0)
    assert_attention_close(out, sdpa_fp32(q, k, v, m), f"plain mask lines {B}x{N}x{S}x{H}x{L} pad {pad}")


def test_dense_op_with_bmc_padded_buffers_and_finfo_min_mask(device):
    """BMC returns padded buffers and pads the mask with finfo.min (cache.py:195-222); the padded
    columns must not contribute."""
    from pace_mi355.llm import BMCKVCache
    from pace_mi355.ops import MultiHeadAttention
    from oracle.attention_ref import causal_mask_4d

    B, H, D, L = 2, 4, 64, 37
    k, v = seeded_kv(8, B, H, L, D)
    cache = BMCKVCache(128)
    K, V = cache.update_cache(k.to(device), v.to(device), 2)
    assert K.shape[2] == 44 and K.is_cuda
    q = seeded_q(9, B, H, 1, D)
    m4 = causal_mask_4d(torch.ones(B, L, dtype=torch.long), 1, L, torch.bfloat16)
    padded = cache.update_mask(m4.to(device), L)
    assert padded.shape[-1] == 44
    out = MultiHeadAttention(dtype=torch.bfloat16)(q.to(device), K, V, attention_mask=padded)
    assert_attention_close(out, sdpa_fp32(q, k, v, m4), "BMC padded")


def test_operator_without_mask_and_noncontiguous_inputs(device):
    from pace_mi355.ops import MultiHeadAttention

    q = seeded_q(1, 2, 8, 4, 16, torch.float32)
    k, v = seeded_kv(2, 2, 8, 4, 16, torch.float32)
    ones = torch.ones(2, 1, 4, 4)  # the reference's operator test passes a mask of ones (test_attention.py:27)
    mha = MultiHeadAttention(dtype=torch.float32)
    out = mha(q.to(device), k.to(device), v.to(device), attention_mask=ones.to(device))
    assert torch.allclose(out.cpu(), sdpa_fp32(q, k, v, ones), atol=1e-3, rtol=1e-3)
    qt = q.transpose(1, 2).contiguous().transpose(1, 2)  # [B,H,S,D] view over [B,S,H,D] storage
    out2 = mha(qt.to(device), k.to(device), v.to(device))
    assert torch.allclose(out2.cpu(), sdpa_fp32(q, k, v), atol=1e-5, rtol=1e-5)


def _random_mask(rng, kind, B, N, S, L, dt):
    """Additive masks of the forms the kernels tell apart; finfo.min marks what is masked."""
    lo = torch.finfo(dt).min
    cols, rows = torch.arange(L)[None, :], torch.arange(S)[:, None]
    heads = N if kind == "per-head" else 1
    m = torch.zeros(B, heads, S, L, dtype=dt)
    if kind in ("causal", "causal-left-padded", "per-head"):
        m = m.masked_fill(cols > rows + (L - S), lo)          # S > L: the first rows read nothing at all
    if kind == "causal-left-padded":
        for b in range(B):
            m[b, :, :, : int(rng.integers(0, max(1, L // 2)))] = lo
    if kind == "window":
        m = m.masked_fill((cols > rows + (L - S)) | (cols < rows + (L - S) - 40), lo)
    if kind == "rows-masked":
        m[:, :, :: int(rng.integers(2, 6)), :] = lo
    if kind == "key-padding":                                  # [B,1,1,L]
        m = torch.zeros(B, 1, 1, L, dtype=dt)
        for b in range(B):
            m[b, :, :, int(rng.integers(1, L + 1)):] = lo
    bias = torch.randn(m.shape, generator=torch.Generator().manual_seed(int(rng.integers(1 << 30)))).to(dt)
    return m + bias * (m == 0)


@pytest.mark.parametrize("seed", range(6))
def test_dense_op_random_shapes_and_masks(device, seed):
    """Seeded sweep over shapes and mask forms, in the spirit of the reference's property test
    (tests/ops/test_sdpa.py:83-127): every kernel the op can take, ragged sizes, masks that leave
    whole stretches (and sometimes whole rows) unreadable."""
    rng = np.random.default_rng(1000 + seed)
    kinds = ["random", "causal", "causal-left-padded", "window", "rows-masked", "per-head", "key-padding"]
    for case in range(8):
        B, N = int(rng.integers(1, 4)), int(rng.integers(1, 10))
        S = int(rng.choice([1, 3, 8, 17, 40, 64, 65, 100, 130, 260]))
        L = int(rng.choice([1, 7, 31, 32, 33, 64, 100, 129, 256, 300]))
        H = int(rng.choice([64, 128, 128, 80, 96, 256]))
        dt = torch.bfloat16
        mdt = torch.bfloat16 if rng.random() < 0.7 else torch.float32
        kind = kinds[int(rng.integers(len(kinds)))]
        q, (k, v) = seeded_q(seed * 100 + case, B, N, S, H), seeded_kv(seed * 100 + case + 50, B, N, L, H)
        m = _random_mask(rng, kind, B, N, S, L, mdt) if kind != "random" else _mask(case, (B, 1, S, L), mdt)
        out = torch.ops.pace.attention(q.to(device), k.to(device), v.to(device), m.to(device), 0)
        assert_attention_close(out, sdpa_fp32(q, k, v, m), f"seed {seed} case {case}: B{B} N{N} S{S} L{L} H{H} {kind} {mdt}")


def test_dense_prefill_is_bit_identical_from_call_to_call(device):
    """The prefill kernel reads V operands from LDS into registers the score products were issued from; before
    those reads were made to wait for the products, one tile's scores differed slightly about once in 300 calls
    of this shape.  Every call must give the same bits."""
    B, N, S, H, L = 2, 32, 512, 64, 128
    k, v = seeded_kv(21, B, N, L, H)
    q = seeded_q(22, B, N, S, H)
    band = (torch.arange(L)[None, :] + torch.arange(S)[:, None]) % 3 == 0
    m = torch.zeros(B, 1, S, L, dtype=torch.bfloat16).masked_fill(band, torch.finfo(torch.bfloat16).min)
    m = m + _mask(23, (B, 1, S, L), torch.bfloat16) * (m == 0)
    qd, kd, vd, md = q.to(device), k.to(device), v.to(device), m.to(device)
    first = torch.ops.pace.attention(qd, kd, vd, md, 0)
    assert_attention_close(first, sdpa_fp32(q, k, v, m), "prefill, banded mask")
    differing = 0
    for _ in range(1500):
        out = torch.ops.pace.attention(qd, kd, vd, md, 0)
        differing += int(not torch.equal(out.view(torch.int16), first.view(torch.int16)))
    assert differing == 0
    # the same through the walk that plain mask lines take (a causal mask: the mask values are not read)
    causal = torch.zeros(B, 1, S, L, dtype=torch.bfloat16).masked_fill(
        torch.arange(L)[None, :] > torch.arange(S)[:, None] // 4, torch.finfo(torch.bfloat16).min)
    cd = causal.to(device)
    first = torch.ops.pace.attention(qd, kd, vd, cd, 0)
    assert_attention_close(first, sdpa_fp32(q, k, v, causal), "prefill, causal mask")
    for _ in range(1000):
        out = torch.ops.pace.attention(qd, kd, vd, cd, 0)
        differing += int(not torch.equal(out.view(torch.int16), first.view(torch.int16)))
    assert differing == 0
    # head_dim 256: the next unit's loads are issued right behind the score products there
    B, N, S, H, L = 2, 16, 256, 256, 128
    k, v = seeded_kv(24, B, N, L, H)
    q = seeded_q(25, B, N, S, H)
    band = (torch.arange(L)[None, :] + torch.arange(S)[:, None]) % 3 == 0
    m = torch.zeros(B, 1, S, L, dtype=torch.bfloat16).masked_fill(band, torch.finfo(torch.bfloat16).min)
    qd, kd, vd, md = q.to(device), k.to(device), v.to(device), m.to(device)
    first = torch.ops.pace.attention(qd, kd, vd, md, 0)
    assert_attention_close(first, sdpa_fp32(q, k, v, m), "prefill, head_dim 256")
    for _ in range(500):
        out = torch.ops.pace.attention(qd, kd, vd, md, 0)
        differing += int(not torch.equal(out.view(torch.int16), first.view(torch.int16)))
    assert differing == 0
