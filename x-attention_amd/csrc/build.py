"""Builds libxattn_hip.so (gfx950) next to its sources with hipcc.

    python x-attention_amd/csrc/build.py

The library is built in-tree so that it travels with the source tree; nothing
is compiled at import time.
"""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
SOURCES = ["capi.hip", "block_sparse_attn.hip", "estimate.hip", "select_blocks.hip", "decode_attn.hip", "profile_threshold.hip", "softmax_block_sum.hip"]
LIB = os.path.join(HERE, "libxattn_hip.so")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Wall",
    "-Wno-unused-result",
    "-Wno-inline-asm",   # the tile copies name M0 (their LDS destination) in an asm clobber list
    "-I" + os.path.join(ROOT, "include"),
    "-I" + HERE,
    # packed fp32 VALU forms are kept out of every kernel
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _run(cmd):
    proc = subprocess.run(cmd, cwd=HERE, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("command failed: " + " ".join(cmd) + "\n" + out)
    return out


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    extra = os.environ.get("XATTN_HIPCC_EXTRA", "").split()
    srcs = [s for s in SOURCES if os.path.exists(os.path.join(HERE, s))]
    objs = [os.path.join(HERE, s.replace(".hip", ".o")) for s in srcs]

    def compile_one(pair):
        src, obj = pair
        return _run([hipcc] + FLAGS + extra + ["-c", src, "-o", obj])

    with ThreadPoolExecutor(max_workers=4) as ex:
        outs = list(ex.map(compile_one, zip(srcs, objs)))
    outs.append(_run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs))
    if verbose:
        for o in outs:
            if o.strip():
                print(o)
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
