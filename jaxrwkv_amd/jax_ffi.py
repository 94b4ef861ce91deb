"""JAX binding of libhiprwkv through XLA custom calls: ``inner_loop`` functions for ``HipRWKV`` classes beside the
reference's ``CudaRWKV`` (/root/reference/src/jaxrwkv/rwkv7.py:450-473, rwkv4.py:386-406).

NOT exercised in this repository's tests: ``jax`` is not installed where they run.  It needs ``jax`` with ROCm
support and ``libhiprwkv_xla.so`` (``python -m jaxrwkv_amd.build --xla-ffi``, handlers in ``csrc/xla_ffi.cc``).  Use::

    from jaxrwkv import rwkv7
    from jaxrwkv_amd import jax_ffi
    class HipRWKV(rwkv7.BaseRWKV):
        inner_loop = classmethod(lambda cls, *args: jax_ffi.wkv7_inner_loop(*args))
    rwkv7.HipRWKV = HipRWKV          # picked by name: get_model(..., rwkv_type="HipRWKV")  (auto.py:62, 89)

Differences from the reference's ``wkv7_cuda`` (rwkv7.py:356-446): no ``s_restore`` residual and no ``T % 16`` /
``T == 1`` special cases; gradients reach ``s`` and come from the returned state; ``new_starts`` is honoured in the
backward pass; batching is ``vmap_method="broadcast_all"`` (every leading axis is one flat batch inside the
handler), so no ``custom_vmap`` rules are needed.  Results equal ``AssociativeScanRWKV`` (``COMPAT_ASSOC``).
"""
import ctypes
import os

import jax
import jax.numpy as jnp
import numpy as np

COMPAT_ASSOC = 1
_LIB = os.path.join(os.path.dirname(os.path.abspath(__file__)), "libhiprwkv_xla.so")
_TARGETS = {"hip-wkv7-fwd": "HipWkv7Fwd", "hip-wkv7-bwd": "HipWkv7Bwd", "hip-wkv6-fwd": "HipWkv6Fwd",
            "hip-wkv6-bwd": "HipWkv6Bwd", "hip-wkv4-fwd": "HipWkv4Fwd", "hip-wkv4-bwd": "HipWkv4Bwd"}
_registered = False


def register():
    """Load the handler library once and register its symbols for the ROCm platform (rwkv7.py:453-465)."""
    global _registered
    if _registered:
        return
    lib = ctypes.cdll.LoadLibrary(_LIB)
    for target, symbol in _TARGETS.items():
        jax.ffi.register_ffi_target(target, jax.ffi.pycapsule(getattr(lib, symbol)), platform="ROCM")
    lib.hiprwkv_wkv7_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.hiprwkv_wkv6_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.hiprwkv_wkv4_bwd_workspace_bytes.restype = ctypes.c_size_t
    for f in (lib.hiprwkv_wkv7_bwd_workspace_bytes, lib.hiprwkv_wkv6_bwd_workspace_bytes):
        f.argtypes = [ctypes.c_int64] * 4
    lib.hiprwkv_wkv4_bwd_workspace_bytes.argtypes = [ctypes.c_int64] * 3
    register.lib = lib
    _registered = True


def _call(target, result_types, *operands):
    # vmap_method="broadcast_all" hands a vmapped call to the handler with the mapped axes as extra LEADING
    # dimensions on every operand (unmapped operands are broadcast to the same leading shape, at the cost of a
    # copy).  The handlers in csrc/xla_ffi.cc rely on exactly that: they take the last three (WKV4: two) dimensions
    # as (T, H, N) and fold everything before them into one flat batch B, for the state, length and new_starts
    # operands too.  An operand vmapped with a non-leading out-axis would break this; jax.ffi never produces one.
    # The per-head / per-channel parameters (WKV6 u (H,N), WKV4 w and u (C,)) then arrive with the same leading batch
    # shape, and the C ABI reads only the first (H,N) / (C,) of them: right when they were broadcast, which is the
    # reference's use (one parameter set per model), and silently wrong for a caller that vmaps over per-example
    # parameters.
    return jax.ffi.ffi_call(target, result_types, vmap_method="broadcast_all")(*operands, flags=np.int64(COMPAT_ASSOC))


def _sds(x, dtype=None):
    return jax.ShapeDtypeStruct(x.shape, dtype or x.dtype)


def _zero_cotangents(length, new_starts):
    # integer / boolean inputs get symbolic-zero cotangents (rwkv7.py:411)
    return np.zeros(np.shape(length), jax.dtypes.float0), np.zeros(np.shape(new_starts), jax.dtypes.float0)


# ------------------------------------------------------------------------------------------------------ WKV7
@jax.custom_vjp
def wkv7_hip(r, w, k, v, a, b, s, length, new_starts):
    return _wkv7_fwd(r, w, k, v, a, b, s, length, new_starts)[0]


def _wkv7_fwd(r, w, k, v, a, b, s, length, new_starts):
    register()
    length = jnp.uint32(length)
    out, sa, new_s = _call("hip-wkv7-fwd", (_sds(r), _sds(r, jnp.float32 if r.dtype == jnp.float32 else jnp.float16), _sds(s)),
                           w, r, k, v, a, b, s, length, new_starts)
    return (new_s, out), (r, w, k, v, a, b, s, length, new_starts, sa)


def _wkv7_bwd(res, grads):
    r, w, k, v, a, b, s, length, new_starts, sa = res
    gs_out, gy = grads
    T, H, N = r.shape[-3:]
    nbytes = register.lib.hiprwkv_wkv7_bwd_workspace_bytes(int(np.prod(r.shape[:-3], dtype=np.int64)), T, H, N)
    ws = jax.ShapeDtypeStruct((nbytes,), jnp.uint8)
    gw, gr, gk, gv, ga, gb, gs, _ = _call("hip-wkv7-bwd", tuple(_sds(x) for x in (w, r, k, v, a, b, s)) + (ws,),
                                          w, r, k, v, a, b, s, length, new_starts, gy, sa, gs_out)
    return (gr, gw, gk, gv, ga, gb, gs) + _zero_cotangents(length, new_starts)


wkv7_hip.defvjp(_wkv7_fwd, _wkv7_bwd)


def wkv7_inner_loop(r, w, k, v, a, b, s, length, new_starts):
    """Signature and return of rwkv7.BaseRWKV.inner_loop (rwkv7.py:200): (new_state, out)."""
    new_s, out = wkv7_hip(r, w, k, v, a, b, s, length, new_starts)
    return new_s.astype(r.dtype), out


# ------------------------------------------------------------------------------------------------------ WKV6
@jax.custom_vjp
def wkv6_hip(r, k, v, w, u, s, length, new_starts):
    return _wkv6_fwd(r, k, v, w, u, s, length, new_starts)[0]


def _wkv6_fwd(r, k, v, w, u, s, length, new_starts):
    register()
    length = jnp.uint32(length)
    out, new_s = _call("hip-wkv6-fwd", (_sds(r), _sds(s)), r, k, v, w, u, s, length, new_starts)
    return (new_s, out), (r, k, v, w, u, s, length, new_starts)


def _wkv6_bwd(res, grads):
    r, k, v, w, u, s, length, new_starts = res
    gs_out, gy = grads
    T, H, N = r.shape[-3:]
    lead = r.shape[:-3]
    nbytes = register.lib.hiprwkv_wkv6_bwd_workspace_bytes(int(np.prod(lead, dtype=np.int64)), T, H, N)
    gu_t = jax.ShapeDtypeStruct(lead + (H, N), jnp.float32)
    gr, gk, gv, gw, gu, gs, _ = _call("hip-wkv6-bwd", (_sds(r), _sds(k), _sds(v), _sds(w), gu_t, _sds(s),
                                                       jax.ShapeDtypeStruct((nbytes,), jnp.uint8)),
                                      r, k, v, w, u, s, length, new_starts, gy, gs_out)
    gu = gu.reshape((-1, H, N)).sum(0).astype(u.dtype).reshape(u.shape)
    return (gr, gk, gv, gw, gu, gs) + _zero_cotangents(length, new_starts)


wkv6_hip.defvjp(_wkv6_fwd, _wkv6_bwd)


def wkv6_inner_loop(r, k, v, w, time_first, s, length, new_starts):
    """rwkv6.BaseRWKV.inner_loop (rwkv6.py:175): w (T,H,N,1) log decay, time_first (H,N,1)."""
    new_s, out = wkv6_hip(r, k, v, w.reshape(r.shape), time_first.reshape(time_first.shape[:2]), s, length, new_starts)
    return new_s.astype(r.dtype), out


# ------------------------------------------------------------------------------------------------------ WKV4
@jax.custom_vjp
def wkv4_hip(w_neg, u, k, v, s, length, new_starts):
    return _wkv4_fwd(w_neg, u, k, v, s, length, new_starts)[0]


def _wkv4_fwd(w_neg, u, k, v, s, length, new_starts):
    register()
    length = jnp.uint32(length)
    new_s, out = _call("hip-wkv4-fwd", (_sds(s), _sds(k)), w_neg, u, k, v, s, length, new_starts)
    return (new_s, out), (w_neg, u, k, v, s, length, new_starts)


def _wkv4_bwd(res, grads):
    w_neg, u, k, v, s, length, new_starts = res
    gs_new, gy = grads
    T, C = k.shape[-2:]
    lead = k.shape[:-2]
    nbytes = register.lib.hiprwkv_wkv4_bwd_workspace_bytes(int(np.prod(lead, dtype=np.int64)), T, C)
    per_seq = jax.ShapeDtypeStruct(lead + (C,), jnp.float32)
    gw, gu, gk, gv, gs, _ = _call("hip-wkv4-bwd", (per_seq, per_seq, _sds(k), _sds(v), _sds(s),
                                                   jax.ShapeDtypeStruct((nbytes,), jnp.uint8)),
                                  w_neg, u, k, v, gy, s, length, new_starts, gs_new)
    gw = gw.reshape((-1, C)).sum(0).astype(w_neg.dtype)          # summed over the batch as in rwkv4.py:351
    gu = gu.reshape((-1, C)).sum(0).astype(u.dtype)
    return (gw, gu, gk, gv, gs) + _zero_cotangents(length, new_starts)


wkv4_hip.defvjp(_wkv4_fwd, _wkv4_bwd)


def wkv4_inner_loop(r, k, v, time_decay, time_first, s, length, new_starts):
    """rwkv4.BaseRWKV.inner_loop (rwkv4.py:144): applies w = -exp(time_decay) (:145, 312) and r * wkv (:163, 406)."""
    new_s, out = wkv4_hip(-jnp.exp(time_decay), time_first, k, v, s, length, new_starts)
    return new_s, r * out
