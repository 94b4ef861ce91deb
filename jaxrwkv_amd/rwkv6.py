"""``HipRWKV`` for RWKV-6: ``inner_loop(cls, r, k, v, w, time_first, s, length, new_starts)`` of
/root/reference/src/jaxrwkv/rwkv6.py:175 (variants :257, :278) served by the gfx950 kernels.  The reference
has no native WKV6 op (README.md:93-99).  ``w`` is the log decay ``-exp(raw)`` with the reference's trailing
singleton axis ``(T,H,N,1)`` (rwkv6.py:217-218) or without it; ``time_first`` is ``(H,N,1)`` or ``(H,N)``."""
import torch

from . import ops


class HipRWKV:
    #: True -> returned state follows AssociativeScanRWKV (rwkv6.py:301); False -> BaseRWKV (rwkv6.py:190)
    assoc_compat = True

    @classmethod
    def inner_loop(cls, r, k, v, w, time_first, s, length, new_starts):
        batched = r.dim() == 4
        if not batched:
            r, k, v, s = (x[None] for x in (r, k, v, s))
            w = w.reshape((1,) + tuple(r.shape[1:]))
            if torch.is_tensor(new_starts) and new_starts.dim() == 1:
                new_starts = new_starts[None]
        else:
            w = w.reshape(r.shape)
        new_s, y = ops.wkv6(r, k, v, w, time_first.reshape(r.shape[2], r.shape[3]), s, length, new_starts,
                            cls.assoc_compat)
        new_s = new_s.to(r.dtype)
        if not batched:
            new_s, y = new_s[0], y[0]
        return new_s, y

    @classmethod
    def step_packed(cls, r, k, v, w, time_first, s, new_s, length, new_starts):
        """``inner_loop`` for a few tokens (T <= 8, decode) with the state read from and written to views of the packed
        model state (``state[:, layer, 2:]`` with a batch axis in front, rwkv6.py:221-224) instead of copies of them;
        batched, no autograd.  Returns ``out``; ``new_s`` is filled in place."""
        return ops.wkv6_step(r, k, v, w.reshape(r.shape), time_first.reshape(r.shape[2], r.shape[3]), s, new_s, length,
                             new_starts, cls.assoc_compat)
