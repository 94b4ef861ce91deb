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
backward pass; every leading axis is one flat batch inside the handler, and a ``custom_vmap`` rule (``_call``) keeps
the per-model parameters (WKV6 ``u``, WKV4 ``w`` and ``u``) un-batched and refuses a vmap over them.  Results equal
``AssociativeScanRWKV`` (``COMPAT_ASSOC``).
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


def _call(target, result_types, *operands, params=()):
    """One XLA custom call.  ``params`` lists the positions of per-model parameters among the operands (WKV6 ``u``
    (H,N), WKV4 ``w`` and ``u`` (C,)): the C ABI takes exactly one set of them per call.

    Batching.  The handlers in csrc/xla_ffi.cc take the last three (WKV4: two) dimensions of the token operands as
    (T, H, N) and fold everything before them into one flat batch, for the state, length and new_starts operands too;
    the parameters must arrive at their own rank.  A plain ``vmap_method="broadcast_all"`` would hand a vmapped call
    the parameters broadcast to the batch shape (or, for a caller that maps over per-example parameters, B different
    sets of which only the first would be read).  The call is therefore wrapped in a ``custom_vmap`` rule that keeps
    the parameters un-batched, broadcasts every other un-mapped operand to the mapped axis (at the cost of a copy,
    as ``broadcast_all`` does), and raises for a vmap over a parameter.  The rule calls the wrapped function again, so
    nested vmaps add one leading axis each."""
    params = tuple(params)

    @jax.custom_batching.custom_vmap
    def call(*ops):
        return tuple(jax.ffi.ffi_call(target, result_types(*ops), vmap_method="broadcast_all")(
            *ops, flags=np.int64(COMPAT_ASSOC)))

    @call.def_vmap
    def _rule(axis_size, in_batched, *ops):
        for i in params:
            if in_batched[i]:
                raise NotImplementedError(
                    f"{target}: operand {i} is a per-model parameter; the kernel takes one set per call, so a vmap "
                    "over it (per-example parameters) is not supported -- loop over the parameter sets instead")
        ops = tuple(x if (bt or i in params) else jnp.broadcast_to(x[None], (axis_size,) + jnp.shape(x))
                    for i, (x, bt) in enumerate(zip(ops, in_batched)))
        outs = call(*ops)
        return outs, tuple(True for _ in outs)

    return call(*operands)


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
    # the residual sa is fp32 beside fp32 I/O and IEEE half beside bf16 I/O (the reference's sa_restore is fp32 for
    # both, rwkv7.py:364); the handlers check the element type against r's
    types = lambda w, r, k, v, a, b, s, length, new_starts: (
        _sds(r), _sds(r, jnp.float32 if r.dtype == jnp.float32 else jnp.float16), _sds(s))
    out, sa, new_s = _call("hip-wkv7-fwd", types, w, r, k, v, a, b, s, length, new_starts)
    return (new_s, out), (r, w, k, v, a, b, s, length, new_starts, sa)


def _wkv7_bwd(res, grads):
    r, w, k, v, a, b, s, length, new_starts, sa = res
    gs_out, gy = grads
    def types(w, r, k, v, a, b, s, length, new_starts, gy, sa, gs_out):
        T, H, N = r.shape[-3:]
        nbytes = register.lib.hiprwkv_wkv7_bwd_workspace_bytes(int(np.prod(r.shape[:-3], dtype=np.int64)), T, H, N)
        return tuple(_sds(x) for x in (w, r, k, v, a, b, s)) + (jax.ShapeDtypeStruct((nbytes,), jnp.uint8),)
    gw, gr, gk, gv, ga, gb, gs, _ = _call("hip-wkv7-bwd", types, w, r, k, v, a, b, s, length, new_starts, gy, sa, gs_out)
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
    types = lambda r, k, v, w, u, s, length, new_starts: (_sds(r), _sds(s))
    out, new_s = _call("hip-wkv6-fwd", types, r, k, v, w, u, s, length, new_starts, params=(4,))
    return (new_s, out), (r, k, v, w, u, s, length, new_starts)


def _wkv6_bwd(res, grads):
    r, k, v, w, u, s, length, new_starts = res
    gs_out, gy = grads
    H, N = r.shape[-2:]

    def types(r, k, v, w, u, s, length, new_starts, gy, gs_out):
        T, H, N = r.shape[-3:]
        lead = r.shape[:-3]
        nbytes = register.lib.hiprwkv_wkv6_bwd_workspace_bytes(int(np.prod(lead, dtype=np.int64)), T, H, N)
        return (_sds(r), _sds(k), _sds(v), _sds(w), jax.ShapeDtypeStruct(lead + (H, N), jnp.float32), _sds(s),
                jax.ShapeDtypeStruct((nbytes,), jnp.uint8))
    gr, gk, gv, gw, gu, gs, _ = _call("hip-wkv6-bwd", types, r, k, v, w, u, s, length, new_starts, gy, gs_out,
                                      params=(4,))
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
    types = lambda w_neg, u, k, v, s, length, new_starts: (_sds(s), _sds(k))
    new_s, out = _call("hip-wkv4-fwd", types, w_neg, u, k, v, s, length, new_starts, params=(0, 1))
    return (new_s, out), (w_neg, u, k, v, s, length, new_starts)


def _wkv4_bwd(res, grads):
    w_neg, u, k, v, s, length, new_starts = res
    gs_new, gy = grads
    C = k.shape[-1]

    def types(w_neg, u, k, v, gy, s, length, new_starts, gs_new):
        T, C = k.shape[-2:]
        lead = k.shape[:-2]
        nbytes = register.lib.hiprwkv_wkv4_bwd_workspace_bytes(int(np.prod(lead, dtype=np.int64)), T, C)
        per_seq = jax.ShapeDtypeStruct(lead + (C,), jnp.float32)
        return (per_seq, per_seq, _sds(k), _sds(v), _sds(s), jax.ShapeDtypeStruct((nbytes,), jnp.uint8))
    gw, gu, gk, gv, gs, _ = _call("hip-wkv4-bwd", types, w_neg, u, k, v, gy, s, length, new_starts, gs_new,
                                  params=(0, 1))
    gw = gw.reshape((-1, C)).sum(0).astype(w_neg.dtype)          # summed over the batch as in rwkv4.py:351
    gu = gu.reshape((-1, C)).sum(0).astype(u.dtype)
    return (gw, gu, gk, gv, gs) + _zero_cotangents(length, new_starts)


wkv4_hip.defvjp(_wkv4_fwd, _wkv4_bwd)


def wkv4_inner_loop(r, k, v, time_decay, time_first, s, length, new_starts):
    """rwkv4.BaseRWKV.inner_loop (rwkv4.py:144): applies w = -exp(time_decay) (:145, 312) and r * wkv (:163, 406)."""
    new_s, out = wkv4_hip(-jnp.exp(time_decay), time_first, k, v, s, length, new_starts)
    return new_s, r * out
