"""Writes the small golden fixtures of this directory from the CPU oracle.

    python tests/golden/make_fixtures.py

Every fixture holds seeded inputs and the oracle's outputs for them (bf16 tensors as their
uint16 bit patterns).  The reference holds no data files for this path, so these vectors come
from the restatement in ``oracle/``, which is pinned by ``tests/test_oracle_*.py``.  The CPU
suite checks that the oracle still reproduces them; the GPU suite checks the HIP path against them.
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import rope_ref  # noqa: E402
from oracle.attention_ref import sdpa_fp32  # noqa: E402
from oracle.cache_ref import DynamicKVCacheRef, repeat_kv  # noqa: E402
from oracle.paged_ref import RaggedCacheModel  # noqa: E402


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def randn_bf16(gen, *shape):
    return torch.randn(*shape, generator=gen).to(torch.bfloat16)


def cache_fixture():
    g = torch.Generator().manual_seed(1234)
    B, H, D, steps = 2, 2, 64, [5, 1, 3, 20]
    ref = DynamicKVCacheRef(64)
    out = {"steps": np.array(steps)}
    for i, T in enumerate(steps):
        k, v = randn_bf16(g, B, H, T, D), randn_bf16(g, B, H, T, D)
        out[f"k{i}"], out[f"v{i}"] = bits(k), bits(v)
        ref.update_cache(k, v, 2)
    ref.remove_cache(4)  # a rollback at the end
    out["key"], out["value"] = bits(ref.key), bits(ref.value)
    return out


def rope_fixture():
    g = torch.Generator().manual_seed(4321)
    B, H, S, D = 2, 3, 5, 64
    x = randn_bf16(g, B, H, S, D)
    pos = torch.tensor([[0, 1, 2, 3, 4], [100, 101, 250, 7, 255]])
    cos, sin, _, _ = rope_ref.cos_sin_tables(
        dict(rope_type="llama3", factor=8.0, low_freq_factor=1.0, high_freq_factor=4.0, original_max_position_embeddings=64),
        D, 256, 500000.0)
    c, s = rope_ref.lookup(cos, sin, pos, torch.bfloat16)
    return {
        "x": bits(x), "positions": pos.numpy(), "cos": cos.numpy(), "sin": sin.numpy(),
        "neox": bits(rope_ref.rotate(x, c, s, neox=True)), "gptj": bits(rope_ref.rotate(x, c, s, neox=False)),
    }


def decode_fixture():
    g = torch.Generator().manual_seed(777)
    B, hkv, n_rep, D = 2, 2, 2, 64
    lens = [37, 20]
    model = RaggedCacheModel(B, hkv, D)
    k, v = randn_bf16(g, B, hkv, max(lens), D), randn_bf16(g, B, hkv, max(lens), D)
    model.append(k, v, lens)
    q1 = randn_bf16(g, B, hkv * n_rep, 1, D)
    q3 = randn_bf16(g, B, hkv * n_rep, 3, D)
    return {
        "lens": np.array(lens), "k": bits(k), "v": bits(v), "q1": bits(q1), "q3": bits(q3), "n_rep": np.array(n_rep),
        "decode": model.attention(q1, n_rep).numpy(), "verify": model.attention(q3, n_rep).numpy(),
    }


FIXTURES = {"cache_append.npz": cache_fixture, "rope.npz": rope_fixture, "paged_attention.npz": decode_fixture}


def main():
    for name, make in FIXTURES.items():
        np.savez_compressed(os.path.join(HERE, name), **make())
        print("wrote", name, os.path.getsize(os.path.join(HERE, name)), "bytes")


if __name__ == "__main__":
    main()
