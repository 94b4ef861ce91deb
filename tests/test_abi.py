"""CPU-only checks of the boundary: the library loads, exports every declared symbol, and refuses CPU tensors."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "hiprwkv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hiprwkv_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    for need in ("hiprwkv_wkv7_fwd", "hiprwkv_wkv7_bwd", "hiprwkv_wkv6_fwd", "hiprwkv_wkv6_bwd", "hiprwkv_wkv4_fwd",
                 "hiprwkv_last_error"):
        assert need in syms


def test_library_exports_every_declared_symbol():
    from jaxrwkv_amd import _lib
    lib = _lib.load()
    for sym in declared_symbols():
        assert hasattr(lib, sym), sym
        assert sym in _lib.SIGNATURES, f"{sym} has no ctypes signature"
    assert lib.hiprwkv_version() >= 100


def test_argument_validation_without_gpu():
    from jaxrwkv_amd import _lib
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    # head size other than 64 and null pointers are refused before anything is launched
    rc = lib.hiprwkv_wkv7_fwd(null, 0, 0, 1, 8, 1, 32, *([null] * 12), 0)
    assert rc == -1 and b"N=32" in lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv7_fwd(null, 0, 0, 1, 8, 1, 64, *([null] * 12), 0)
    assert rc == -1 and b"null" in lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv6_fwd(null, 7, 0, 1, 8, 1, 64, *([null] * 10), 0)
    assert rc == -1 and b"dtype" in lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv4_fwd(null, 0, 0, 8, 64, *([null] * 9), 0)
    assert rc == -1
    # WKV4 channel limit (32-bit byte offsets inside a block of tokens), forward and backward
    rc = lib.hiprwkv_wkv4_fwd(null, 0, 1, 8, (1 << 23) + 1, *([null] * 9), 0)
    assert rc == -1 and b"2^23" in lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv4_bwd(null, 0, 1, 8, (1 << 23) + 1, *([null] * 14), null, 0, 0)
    assert rc == -1 and b"2^23" in lib.hiprwkv_last_error()
    assert lib.hiprwkv_wkv4_bwd_workspace_bytes(2, 17, 64) >= 2 * 2 * 3 * 64 * 4
    # the forward that keeps the backward's checkpoints: workspace pointer and size are checked first
    ok = ctypes.c_void_p(0x10000)
    rc = lib.hiprwkv_wkv4_fwd_ckpt(null, 0, 2, 17, 64, *([ok] * 5), null, null, ok, ok, null, 1 << 20, 0)
    assert rc == -1 and b"workspace" in lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv4_fwd_ckpt(null, 0, 2, 17, 64, *([ok] * 5), null, null, ok, ok, ok, 16, 0)
    assert rc == -3 and b"needed" in lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv4_fwd_ckpt(null, 0, 0, 17, 64, *([ok] * 5), null, null, ok, ok, ok, 1 << 20, 0)
    assert rc == -1
    # three fp32 (B,T,H,N) arrays, each with 1 KiB of room to start at its own 128-byte phase
    assert lib.hiprwkv_wkv7_bwd_workspace_bytes(2, 16, 2, 64) == 3 * (2 * 16 * 2 * 64 * 4 + 1024)
    # the decode step on a packed state: at most 8 tokens, batch strides of at least one state and 16-byte multiples
    step = lambda T, s_stride, o_stride, st=1: lib.hiprwkv_wkv7_step(null, 1, st, 2, T, 2, 64, *([ok] * 7), s_stride, null,
                                                                   null, ok, ok, o_stride, 0)
    assert step(9, 8192, 8192) == -1 and b"at most 8" in lib.hiprwkv_last_error()
    assert step(1, 8191, 8192) == -1 and b"less than" in lib.hiprwkv_last_error()
    assert step(1, 8192, 8192 + 4) == -1 and b"16 bytes" in lib.hiprwkv_last_error()
    assert step(1, 8192 + 2, 8192, st=0) == -1 and b"16 bytes" in lib.hiprwkv_last_error()
    step6 = lambda T, s_stride, o_stride: lib.hiprwkv_wkv6_step(null, 1, 1, 2, T, 2, 64, *([ok] * 6), s_stride, null, null, ok,
                                                                ok, o_stride, 0)
    assert step6(9, 8192, 8192) == -1 and b"at most 8" in lib.hiprwkv_last_error()
    assert step6(1, 8192, 100) == -1 and b"less than" in lib.hiprwkv_last_error()
    assert lib.hiprwkv_wkv6_bwd_workspace_bytes(2, 16, 2, 64) >= 2 * 16 * 2 * 64 * 4


def test_misaligned_pointers_are_refused_by_every_entry_point():
    """All tensor pointers must be 16-byte aligned (the kernels use 8- and 16-byte accesses); refused before a launch."""
    from jaxrwkv_amd import _lib
    lib = _lib.load()
    ok, bad, null = ctypes.c_void_p(0x10000), ctypes.c_void_p(0x10008), ctypes.c_void_p(0)
    msg = lambda: lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv7_fwd(null, 1, 0, 1, 32, 1, 64, ok, ok, bad, ok, ok, ok, ok, null, null, ok, null, ok, 0)
    assert rc == -1 and b"aligned" in msg()
    rc = lib.hiprwkv_wkv6_fwd(null, 1, 0, 1, 32, 1, 64, ok, ok, ok, bad, ok, ok, null, null, ok, ok, 0)
    assert rc == -1 and b"aligned" in msg()
    rc = lib.hiprwkv_wkv4_fwd(null, 0, 1, 8, 64, ok, ok, bad, ok, ok, null, null, ok, ok, 0)
    assert rc == -1 and b"aligned" in msg()
    rc = lib.hiprwkv_wkv4_bwd(null, 0, 1, 8, 64, ok, ok, ok, ok, ok, ok, null, null, null, ok, ok, ok, bad, ok, ok, 1 << 20, 0)
    assert rc == -1 and b"aligned" in msg()
    rc = lib.hiprwkv_rwkv7_premix(null, 1, 8, 1, 64, ok, ok, ok, ok, ok, bad, ok)
    assert rc == -1 and b"aligned" in msg()
    rc = lib.hiprwkv_rwkv7_premix_bwd(null, 1, 8, 1, 64, ok, ok, ok, ok, ok, ok, ok, ok, ok, ok, bad)
    assert rc == -1 and b"aligned" in msg()
    rc = lib.hiprwkv_rwkv7_premix_bwd(null, 1, 8, 1, 64, ok, ok, ok, ok, ok, ok, ok, ok, ok, null, ok)
    assert rc == -1 and b"null" in msg()
    rc = lib.hiprwkv_rwkv7_postmix_bwd(null, 1, 8, 1, 64, *([ok] * 8), 1e-5, ok, ok, bad, ok, ok, ok, ok, ok, ok)
    assert rc == -1 and b"aligned" in msg()
    rc = lib.hiprwkv_rwkv7_postmix_bwd(null, 1, 8, 1, 32, *([ok] * 8), 1e-5, *([ok] * 9))
    assert rc == -1 and b"N=32" in msg()
    rc = lib.hiprwkv_rwkv7_postmix(null, 1, 8, 1, 64, ok, bad, ok, ok, ok, ok, ok, ok, 1e-5, ok)
    assert rc == -1 and b"aligned" in msg()
    # decay / gate / value mix between the projections and the op
    assert lib.hiprwkv_rwkv7_decay(null, 1, 8, 64, ok, bad, ok) == -1 and b"aligned" in msg()
    assert lib.hiprwkv_rwkv7_decay(null, 1, 8, 60, ok, ok, ok) == -1 and b"multiple of 8" in msg()
    assert lib.hiprwkv_rwkv7_decay_bwd(null, 1, 8, 64, ok, ok, ok, ok, null) == -1 and b"null" in msg()
    assert lib.hiprwkv_rwkv7_agate(null, 7, 8, 64, ok, ok, ok) == -1 and b"dtype" in msg()
    assert lib.hiprwkv_rwkv7_agate_bwd(null, 1, 0, 64, ok, ok, ok, ok, ok) == -1 and b"positive" in msg()
    assert lib.hiprwkv_rwkv7_relusq(null, 1, 60, ok, ok) == -1 and b"multiple of 8" in msg()
    assert lib.hiprwkv_rwkv7_relusq_bwd(null, 1, 64, ok, bad, ok) == -1 and b"aligned" in msg()
    assert lib.hiprwkv_rwkv7_vmix(null, 1, 8, 64, ok, ok, ok, ok, bad) == -1 and b"aligned" in msg()
    assert lib.hiprwkv_rwkv7_vmix_bwd(null, 1, 8, 64, ok, ok, ok, ok, ok, ok, bad, ok, ok) == -1 and b"aligned" in msg()
    # token shift + interpolation: pointer arrays in host memory, C a multiple of 8, one or six outputs
    arr = lambda *ps: (ctypes.c_void_p * len(ps))(*[p.value for p in ps])
    six_ok, six_bad = arr(*([ok] * 6)), arr(ok, ok, ok, bad, ok, ok)
    assert lib.hiprwkv_rwkv7_shiftmix(null, 1, 2, 8, 64, 6, ok, ok, 64, null, six_ok, six_bad) == -1 and b"aligned" in msg()
    assert lib.hiprwkv_rwkv7_shiftmix(null, 1, 2, 8, 60, 6, ok, ok, 64, null, six_ok, six_ok) == -1 and b"multiple of 8" in msg()
    assert lib.hiprwkv_rwkv7_shiftmix(null, 1, 2, 8, 64, 3, ok, ok, 64, null, six_ok, six_ok) == -1 and b"n_out" in msg()
    assert lib.hiprwkv_rwkv7_shiftmix(null, 1, 2, 8, 64, 1, ok, ok, 60, null, six_ok, six_ok) == -1 and b"stride" in msg()
    assert lib.hiprwkv_rwkv7_shiftmix(null, 1, 2, 8, 64, 1, ok, null, 64, null, six_ok, six_ok) == -1 and b"null" in msg()
    assert lib.hiprwkv_rwkv7_shiftmix_bwd(null, 1, 2, 8, 64, 6, ok, ok, 64, null, six_ok, six_bad, ok, ok, 64, ok) == -1
    assert lib.hiprwkv_rwkv7_shiftmix_bwd(null, 1, 2, 8, 64, 6, ok, ok, 64, null, six_ok, six_ok, ok, ok, 64, null) == -1 and b"null" in msg()
    assert lib.hiprwkv_rwkv7_shiftmix_bwd(null, 1, 2, 8, 64, 6, ok, ok, 64, null, six_ok, six_ok, ok, ok, 12, ok) == -1 and b"dprev" in msg()


def test_cpu_tensors_are_refused_loudly():
    from jaxrwkv_amd import _lib, ops
    x = torch.zeros(1, 4, 1, 64)
    with pytest.raises(_lib.HipRwkvError):
        ops.wkv7_fwd(x, x, x, x, x, x, torch.zeros(1, 1, 64, 64))
    with pytest.raises(_lib.HipRwkvError):
        ops.wkv4_fwd(torch.zeros(8), torch.zeros(8), torch.zeros(1, 4, 8), torch.zeros(1, 4, 8), torch.zeros(1, 3, 8))


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "jaxrwkv_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src, f"{f} mentions the oracle"


def test_xla_ffi_sources_agree_on_symbols_and_abi():
    """The XLA handler translation unit cannot be compiled here (no XLA headers): check statically that the Python
    binding registers exactly the handler symbols it defines and that it only calls functions the C ABI declares."""
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cc = open(os.path.join(root, "jaxrwkv_amd", "csrc", "xla_ffi.cc")).read()
    py = open(os.path.join(root, "jaxrwkv_amd", "jax_ffi.py")).read()
    header = open(os.path.join(root, "include", "hiprwkv.h")).read()
    defined = set(re.findall(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\((\w+),", cc))
    registered = set(re.findall(r'"hip-wkv\d-(?:fwd|bwd)": "(\w+)"', py))
    assert defined == registered and len(defined) == 6
    for fn in set(re.findall(r"\b(hiprwkv_\w+)\(", cc)):
        assert re.search(r"\b%s\(" % fn, header), fn
    # Each handler's parameter list and its binding declare the same number of buffers, in the same kinds.
    for name in defined:
        fn = name.replace("Hip", "")
        params = re.search(r"ffi::Error %s\(hipStream_t stream,(.*?)\) \{" % fn, cc, re.S).group(1)
        bind = re.search(r"XLA_FFI_DEFINE_HANDLER_SYMBOL\(%s, %s,(.*?)\);" % (name, fn), cc, re.S).group(1)
        p_args = re.findall(r"ffi::(AnyBuffer|Buffer<ffi::\w+>) \w+", re.sub(r"ffi::Result<ffi::(?:AnyBuffer|Buffer<ffi::\w+>)> \w+", "", params))
        p_rets = re.findall(r"ffi::Result<ffi::(AnyBuffer|Buffer<ffi::\w+>)> \w+", params)
        b_args = re.findall(r"\.Arg<ffi::(AnyBuffer|Buffer<ffi::\w+>)>\(\)", bind)
        b_rets = re.findall(r"\.Ret<ffi::(AnyBuffer|Buffer<ffi::\w+>)>\(\)", bind)
        assert p_args == b_args, (name, p_args, b_args)
        assert p_rets == b_rets, (name, p_rets, b_rets)
    # The WKV7 residual is half beside bf16 I/O: both handlers check its element type against r's, the token operands
    # against each other, and the binding declares the matching result type.
    assert cc.count("sa_type_ok(r.element_type()") == 2 and "io == ffi::BF16 && sa == ffi::F16" in cc
    assert "jnp.float32 if r.dtype == jnp.float32 else jnp.float16" in py
    # Per-model parameters must arrive un-batched: rank checks in the handlers, a custom_vmap rule in the binding.
    assert cc.count("one parameter set per call") >= 4
    assert "custom_vmap" in py and "params=(4,)" in py and "params=(0, 1)" in py
    # The debug hook cannot come in through the XLA attribute.
    assert "static_cast<unsigned>(flags) & HIPRWKV_PUBLIC_FLAGS" in cc and cc.count("public_flags(flags)") == 6


def test_flag_bits_are_validated_without_gpu():
    """Unknown flag bits are refused; the debug hook is refused unless the process environment enables it (checked in
    a child process, because the library reads the variable once); the entry point that allocates nothing refuses
    HIPRWKV_CKPT_READY (its scratch array is shared between calls)."""
    import subprocess
    import sys
    from jaxrwkv_amd import _lib
    lib = _lib.load()
    null = ctypes.c_void_p(0)
    rc = lib.hiprwkv_wkv7_fwd(null, 0, 0, 1, 8, 1, 64, *([null] * 12), 0x4000)
    assert rc == -1 and b"unknown flag" in lib.hiprwkv_last_error()
    rc = lib.hiprwkv_wkv4_fwd(null, 0, 1, 8, 64, *([null] * 9), 0x8)
    assert rc == -1 and b"unknown flag" in lib.hiprwkv_last_error()
    ok = ctypes.c_void_p(0x10000)
    rc = lib.hiprwkv_wkv4_bwd_noalloc(null, 0, 1, 8, 64, *([ok] * 6), null, null, null, *([ok] * 5), _lib.CKPT_READY)
    assert rc == -1 and b"CKPT_READY" in lib.hiprwkv_last_error()
    code = ("import ctypes; from jaxrwkv_amd import _lib; lib = _lib.load(); n = ctypes.c_void_p(0); "
            "rc = lib.hiprwkv_wkv7_fwd(n, 0, 0, 1, 8, 1, 64, *([n] * 12), 0x100); "
            "print(rc, lib.hiprwkv_last_error().decode())")
    for enable, want in ((None, "HIPRWKV_ENABLE_DEBUG_FLAGS"), ("1", "null tensor pointer")):
        env = {k: v for k, v in os.environ.items() if k != "HIPRWKV_ENABLE_DEBUG_FLAGS"}
        if enable:
            env["HIPRWKV_ENABLE_DEBUG_FLAGS"] = enable
        out = subprocess.run([sys.executable, "-c", code], cwd=ROOT, env=env, capture_output=True, text=True, timeout=120)
        assert out.returncode == 0, out.stderr
        assert out.stdout.startswith("-1 ") and want in out.stdout, out.stdout


def test_phased_allocation_gives_the_asked_address_phase():
    """The operators place the large arrays they allocate at distinct 128-byte steps past a 1 KiB boundary
    (jaxrwkv_amd/ops.py); small ones are allocated plainly.  Runs on CPU tensors: only addresses are looked at."""
    import torch
    from jaxrwkv_amd import ops
    ref = torch.empty((2, 512, 8, 64), dtype=torch.bfloat16)            # 1 MiB
    seen = set()
    for steps in range(1, 9):
        t = ops._empty_like_phased(ref, steps)
        assert t.shape == ref.shape and t.dtype == ref.dtype and t.is_contiguous()
        assert (ops._phase(t) - ops._phase(ref)) % 8 == steps % 8
        assert t.data_ptr() % 16 == 0
        seen.add(ops._phase(t))
        t.fill_(1.0)                                                    # the whole view is writable memory
    assert len(seen) == 8
    small = ops._empty_phased((4, 1, 8, 64), torch.float32, "cpu", 3)
    assert small.shape == (4, 1, 8, 64) and small._base is None
    f16 = ops._empty_phased((2, 512, 8, 64), torch.float16, "cpu", 5)
    assert ops._phase(f16) == 5 and f16.dtype == torch.float16
