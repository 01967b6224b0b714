"""Build librwkv_hip.so (gfx950) in-tree with hipcc.

``python -m rwkvstic_amd.build`` or ``build()``; hipcc cross-compiles without a
GPU.  The library is written next to this file so it travels with the tree.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "librwkv_hip.so")
SOURCES = ["rwkv_quant.hip", "rwkv_ops.hip", "rwkv_model.hip", "rwkv_decode.hip", "rwkv_rows.hip", "rwkv_sample.hip"]

FLAGS = [
    "-O3", "-std=c++17", "-fPIC", "-shared",
    "--offload-arch=gfx950",
    # scalar/float2 code must not be turned into packed-fp32 instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def build(verbose: bool = True, extra_flags=(), output: str | None = None) -> str:
    """output: write the library there instead of next to this file (diagnostic builds, e.g. with
    ``-DRWKV_DIAG``, the library's one diagnostic switch: weights of the single-token kernel served from cache, results wrong; ``bench.py --lib`` loads such a file)."""
    srcs = [os.path.join(CSRC, s) for s in SOURCES]
    out = os.path.abspath(output) if output else LIB
    tmp = out + ".tmp"
    cmd = [hipcc(), *FLAGS, *extra_flags, "-o", tmp, *srcs]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    os.replace(tmp, out)
    return out


if __name__ == "__main__":
    import argparse

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--define", action="append", default=[], metavar="NAME[=VALUE]", help="preprocessor definition (repeatable)")
    ap.add_argument("--output", default=None, help="library file to write (default: in-tree librwkv_hip.so)")
    ns = ap.parse_args()
    print(build(extra_flags=[f"-D{d}" for d in ns.define], output=ns.output))
