"""``HipRWKV`` for RWKV-7: the ``inner_loop`` plug-in of the reference, served by the gfx950 kernels.

The reference picks the recurrence implementation by class name (``getattr(rwkv7, rwkv_type)``,
/root/reference/src/jaxrwkv/auto.py:62,89); every variant overrides only
``inner_loop(cls, r, w, k, v, a, b, s, length, new_starts)`` (/root/reference/src/jaxrwkv/rwkv7.py:200, 296, 321, 468).
This class has that signature and return convention ``(new_state, out)`` cast to ``r.dtype`` (rwkv7.py:346).
Differences from the reference's ``CudaRWKV`` (rwkv7.py:450-473), all on purpose: any ``T`` (no multiple-of-16
rule, ``T == 1`` handled natively), gradients flow into ``s`` and back from the returned state, ``new_starts`` is
honoured in the backward pass, and the state is carried in fp32 inside the kernel whatever the I/O dtype.
"""
import torch

from . import ops


class HipRWKV:
    #: True -> results equal AssociativeScanRWKV (rwkv7.py:321-346); False -> BaseRWKV/ScanRWKV (rwkv7.py:200-220)
    assoc_compat = True
    #: True -> the sequential fp32 kernels whatever the dtype (the cross-check of the chunked MFMA kernels)
    force_seq = False

    @classmethod
    def inner_loop(cls, r, w, k, v, a, b, s, length, new_starts):
        """r,w,k,v,a,b ``(T,H,N)`` and s ``(H,N,N)`` as in the reference, or the same with a leading batch axis
        (the reference's ``jax.vmap``; ``length``/``new_starts`` may then be unbatched and are broadcast,
        rwkv7.py:422-427).  Differentiable w.r.t. r,w,k,v,a,b,s."""
        batched = r.dim() == 4
        if not batched:
            r, w, k, v, a, b, s = (x[None] for x in (r, w, k, v, a, b, s))
            if torch.is_tensor(new_starts) and new_starts.dim() == 1:
                new_starts = new_starts[None]
        new_s, y = ops.wkv7(r, w, k, v, a, b, s, length, new_starts, cls.assoc_compat, cls.force_seq)
        new_s = new_s.to(r.dtype)
        if not batched:
            new_s, y = new_s[0], y[0]
        return new_s, y

    @classmethod
    def step_packed(cls, r, w, k, v, a, b, s, new_s, length, new_starts):
        """``inner_loop`` for a few tokens (T <= 8, decode) with the state read from and written to views of the packed
        model state (``state[:, layer, 2:]``, rwkv7.py:254-260) instead of copies of them; batched, no autograd.
        Returns ``out``; ``new_s`` is filled in place."""
        return ops.wkv7_step(r, w, k, v, a, b, s, new_s, length, new_starts, cls.assoc_compat)
