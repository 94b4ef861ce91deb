"""``HipRWKV`` for RWKV-4: ``inner_loop(cls, r, k, v, w, time_first, s, length, new_starts)`` of
/root/reference/src/jaxrwkv/rwkv4.py:144 (variants :217, :253, :402) served by the gfx950 kernel.
As in the reference's ``CudaRWKV`` (rwkv4.py:402-406) the op receives ``-exp(w)`` and the receptance is applied
to its output here.  Differentiable w.r.t. r, k, v, w, time_first and s."""
import torch

from . import ops


class HipRWKV:
    assoc_compat = True

    @classmethod
    def inner_loop(cls, r, k, v, w, time_first, s, length, new_starts):
        """r,k,v ``(T,C)``, w,time_first ``(C,)``, s ``(3,C)`` -- or with a leading batch axis on r,k,v,s."""
        batched = r.dim() == 3
        if not batched:
            r, k, v, s = (x[None] for x in (r, k, v, s))
            if torch.is_tensor(new_starts) and new_starts.dim() == 1:
                new_starts = new_starts[None]
        new_s, wkv = ops.wkv4(-torch.exp(w.float()).to(k.dtype), time_first, k, v, s, length, new_starts,
                              cls.assoc_compat)
        out = r * wkv
        if not batched:
            new_s, out = new_s[0], out[0]
        return new_s, out
