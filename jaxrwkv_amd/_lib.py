"""ctypes binding of ``libhiprwkv.so`` (the C ABI declared in ``include/hiprwkv.h``).

There is no fallback: if the library has not been built, or a call fails, an exception is raised.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libhiprwkv.so")

F32, BF16 = 0, 1
COMPAT_ASSOC = 1
FORCE_SEQ = 2
NO_SMALL_T = 4
W_PER_HEAD = 0x10
CKPT_READY = 0x20
DEBUG_DROP_PUBLISH = 0x100      # refused unless the process runs with HIPRWKV_ENABLE_DEBUG_FLAGS=1
PUBLIC_FLAGS = COMPAT_ASSOC | FORCE_SEQ | NO_SMALL_T | W_PER_HEAD | CKPT_READY

_vp, _i64, _int, _u32, _sz = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_uint, ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/hiprwkv.h declaration by declaration
SIGNATURES = {
    "hiprwkv_last_error": (ctypes.c_char_p, []),
    "hiprwkv_version": (_int, []),
    "hiprwkv_handshake_failures": (_int, [_vp, ctypes.POINTER(ctypes.c_uint)]),
    "hiprwkv_numeric_events": (_int, [_vp, ctypes.POINTER(ctypes.c_uint)]),
    "hiprwkv_wkv7_fwd": (_int, [_vp, _int, _int, _i64, _i64, _i64, _i64] + [_vp] * 7 + [_vp, _vp] + [_vp, _vp, _vp, _u32]),
    "hiprwkv_wkv7_step": (_int, [_vp, _int, _int, _i64, _i64, _i64, _i64] + [_vp] * 6 + [_vp, _i64] + [_vp, _vp]
                          + [_vp, _vp, _i64, _u32]),
    "hiprwkv_wkv7_bwd_workspace_bytes": (_sz, [_i64] * 4),
    "hiprwkv_wkv7_bwd": (_int, [_vp, _int, _int, _i64, _i64, _i64, _i64] + [_vp] * 7 + [_vp, _vp] + [_vp] * 3
                         + [_vp] * 7 + [_vp, _sz, _u32]),
    "hiprwkv_wkv6_fwd": (_int, [_vp, _int, _int, _i64, _i64, _i64, _i64] + [_vp] * 6 + [_vp, _vp] + [_vp, _vp, _u32]),
    "hiprwkv_wkv6_step": (_int, [_vp, _int, _int, _i64, _i64, _i64, _i64] + [_vp] * 5 + [_vp, _i64] + [_vp, _vp]
                          + [_vp, _vp, _i64, _u32]),
    "hiprwkv_wkv6_bwd_workspace_bytes": (_sz, [_i64] * 4),
    "hiprwkv_wkv6_bwd": (_int, [_vp, _int, _int, _i64, _i64, _i64, _i64] + [_vp] * 6 + [_vp, _vp] + [_vp, _vp]
                         + [_vp] * 6 + [_vp, _sz, _u32]),
    "hiprwkv_wkv4_fwd": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 5 + [_vp, _vp] + [_vp, _vp, _u32]),
    "hiprwkv_wkv4_fwd_ckpt": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 5 + [_vp, _vp] + [_vp, _vp, _vp,
                                     ctypes.c_size_t, _u32]),
    "hiprwkv_wkv4_bwd_workspace_bytes": (_sz, [_i64] * 3),
    "hiprwkv_wkv4_bwd": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 6 + [_vp, _vp] + [_vp] + [_vp] * 5
                         + [_vp, _sz, _u32]),
    "hiprwkv_wkv4_bwd_noalloc_max_bytes": (_sz, []),
    "hiprwkv_wkv4_bwd_noalloc": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 6 + [_vp, _vp] + [_vp] + [_vp] * 5 + [_u32]),
    "hiprwkv_rwkv7_shiftmix": (_int, [_vp, _int, _i64, _i64, _i64, _int, _vp, _vp, _i64, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_shiftmix_bwd": (_int, [_vp, _int, _i64, _i64, _i64, _int, _vp, _vp, _i64, _vp, _vp, _vp, _vp, _vp, _i64, _vp]),
    "hiprwkv_rwkv7_decay": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_decay_bwd": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_agate": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_agate_bwd": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_relusq": (_int, [_vp, _int, _i64, _vp, _vp]),
    "hiprwkv_rwkv7_relusq_bwd": (_int, [_vp, _int, _i64, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_vmix": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_vmix_bwd": (_int, [_vp, _int, _i64, _i64, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "hiprwkv_rwkv7_premix": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 7),
    "hiprwkv_rwkv7_postmix": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 8 + [ctypes.c_float, _vp]),
    "hiprwkv_rwkv7_premix_bwd": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 11),
    "hiprwkv_rwkv7_postmix_bwd": (_int, [_vp, _int, _i64, _i64, _i64] + [_vp] * 8 + [ctypes.c_float] + [_vp] * 9),
}

_lib = None


class HipRwkvError(RuntimeError):
    pass


def load():
    """Loads the library once and types every entry point; raises if it is missing."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HipRwkvError(
            f"{LIB_PATH} is missing: build it with `python -m jaxrwkv_amd.build` (there is no CPU fallback)")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(rc, what):
    if rc != 0:
        msg = load().hiprwkv_last_error().decode()
        raise HipRwkvError(f"{what} failed with code {rc}: {msg}")
