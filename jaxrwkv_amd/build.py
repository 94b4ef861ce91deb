"""Compiles the HIP sources under ``csrc/`` into ``jaxrwkv_amd/libhiprwkv.so`` for gfx950.

Run as ``python -m jaxrwkv_amd.build``.  hipcc cross-compiles, so no GPU is needed to build.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhiprwkv.so")
SOURCES = ["api.hip", "wkv7_seq.hip", "wkv7_chunk.hip", "wkv7_chunk_bwd_b.hip", "wkv7_chunk_bwd_c.hip", "wkv7_small_t.hip", "wkv6_seq.hip", "wkv6_chunk.hip", "wkv4.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc",
    # packed-fp32 VALU forms are switched off on purpose for this GPU pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build(verbose=True):
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + FLAGS + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", LIB]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB


if __name__ == "__main__":
    build()
    sys.exit(0)
