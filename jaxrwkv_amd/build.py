"""Compiles the HIP sources under ``csrc/`` into ``jaxrwkv_amd/libhiprwkv.so`` for gfx950.

Run as ``python -m jaxrwkv_amd.build``.  hipcc cross-compiles, so no GPU is needed to build.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB = os.path.join(HERE, "libhiprwkv.so")
SOURCES = ["api.hip", "wkv7_seq.hip", "wkv7_fwd.hip", "wkv7_fwd_f32.hip", "wkv7_bwd_a.hip", "wkv7_chunk_bwd_b.hip", "wkv7_chunk_bwd_c.hip", "wkv7_bwd_a_f32.hip", "wkv7_bwd_b_f32.hip", "wkv7_bwd_c_f32.hip", "wkv7_small_t.hip", "wkv6_seq.hip", "wkv6_small_t.hip", "wkv6_fwd.hip", "wkv6_fwd_f32.hip", "wkv6_chunk_bwd_f.hip", "wkv6_chunk_bwd_r.hip", "wkv6_bwd_f_f32.hip", "wkv6_bwd_r_f32.hip", "wkv4.hip", "rwkv7_mix.hip", "rwkv7_shift.hip", "rwkv7_gates.hip"]
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared", "-fno-gpu-rdc",
    # packed-fp32 VALU forms are switched off on purpose for this GPU pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def build(verbose=True, jobs=None):
    """Compiles every source to an object under ``jaxrwkv_amd/build/`` (in parallel), checks the assembly of each
    (``mfma_hazard``) and links the shared library."""
    from concurrent.futures import ThreadPoolExecutor
    from . import mfma_hazard
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    objdir = os.path.join(HERE, "build")
    os.makedirs(objdir, exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"]

    def run(cmd):
        if verbose:
            print(" ".join(cmd), flush=True)
        res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
        if res.returncode != 0:
            raise RuntimeError("hipcc failed:\n" + out)
        if verbose and out.strip():
            print(out)

    def compile_one(src):
        stem = os.path.join(objdir, os.path.splitext(src)[0])
        run([hipcc] + compile_flags + ["-c", os.path.join(CSRC, src), "-o", stem + ".o"])
        # the same device code as assembly, for the check of MFMA pairings the compiler does not space out
        run([hipcc] + [f for f in compile_flags if f != "-fPIC"] + ["-S", "--cuda-device-only", os.path.join(CSRC, src),
                                                                   "-o", stem + ".s"])
        with open(stem + ".s") as f:
            mfma_hazard.check(f.read(), src)
        return stem + ".o"

    jobs = jobs or min(8, os.cpu_count() or 1)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(compile_one, SOURCES))
    run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc"] + objs + ["-o", LIB])
    return LIB


def build_xla_ffi(verbose=True):
    """Compile csrc/xla_ffi.cc (the XLA custom-call handlers) into libhiprwkv_xla.so next to libhiprwkv.so.
    Needs the XLA FFI headers that ship with jax (``jax.ffi.include_dir()``); raises where jax is not installed."""
    import jax  # noqa: F401  (only here: the rest of the package does not depend on jax)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    out = os.path.join(HERE, "libhiprwkv_xla.so")
    cmd = [hipcc, "-O2", "-std=c++17", "-fPIC", "-shared", "-x", "hip", "--offload-arch=gfx950",
           "-I" + jax.ffi.include_dir(), os.path.join(CSRC, "xla_ffi.cc"), "-L" + HERE, "-l:libhiprwkv.so",
           "-Wl,-rpath,$ORIGIN", "-o", out]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return out


if __name__ == "__main__":
    build()
    if "--xla-ffi" in sys.argv[1:]:
        build_xla_ffi()
    sys.exit(0)
