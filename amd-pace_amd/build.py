"""Build the gfx950 shared library of the KV-cache hot path with hipcc.

    python amd-pace_amd/build.py            # compile + link (always recompiles)

Produces ``amd-pace_amd/pace_mi355/_lib/libpace_kv_hip.so``.  hipcc cross-compiles
for gfx950 without a GPU, so this runs on a CPU-only machine.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
REPO = os.path.dirname(HERE)
CSRC = os.path.join(HERE, "csrc")
OUT_DIR = os.path.join(HERE, "pace_mi355", "_lib")
LIB = os.path.join(OUT_DIR, "libpace_kv_hip.so")
SOURCES = ["common.cpp", "block_plan.cpp", "kv_ops.hip", "rope.hip", "paged_attn.hip", "dense_attn_mfma.hip", "dense_attn.hip"]

FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I", os.path.join(REPO, "include"),
    "-I", CSRC,
]


# Per-source additions.  dense_attn.hip: its fp32 kernels rescale their accumulators in most tiles of a short row,
# and vector instructions cannot take the accumulation registers the compiler otherwise puts matrix results in:
# every rescale then moves 36 registers out and back (measured +4 % on the fp32 prefill shapes; nothing on the others).
SOURCE_FLAGS = {"dense_attn.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"]}


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the gfx950 library cannot be built")
    return exe


def _compile(src: str, obj_dir: str, extra) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [hipcc(), "-x", "hip", "-c", os.path.join(CSRC, src), "-o", obj] + FLAGS + SOURCE_FLAGS.get(src, []) + list(extra)
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "packed-fp32-ops"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed on {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(extra_flags=(), verbose: bool = True) -> str:
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    os.makedirs(OUT_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=4) as pool:
        objs = list(pool.map(lambda s: _compile(s, obj_dir, extra_flags), SOURCES))
    tmp = LIB + ".tmp"
    cmd = [hipcc(), "-shared", "-fPIC", "--offload-arch=gfx950", "-fno-gpu-rdc", "-o", tmp] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB)
    if verbose:
        print(f"built {LIB} ({os.path.getsize(LIB)} bytes)")
    return LIB


if __name__ == "__main__":
    build(sys.argv[1:])
