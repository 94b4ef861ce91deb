"""``HipRWKV`` for RWKV-5 and RWKV-5.2: ``inner_loop(cls, r, k, v, w, time_first, s, length, new_starts)`` of
/root/reference/src/jaxrwkv/rwkv5.py:162-181 and rwkv5_2.py:164-183, served by the WKV6 kernels.

RWKV-5 is the WKV6 recurrence with a decay that does not depend on the token: ``w`` is the decay itself
(``exp(-exp(time_decay))``), one value per head ``(H,1,1)`` (rwkv5.py:194) or per head channel ``(H,N,1)``
(rwkv5_2.py:198); ``time_first`` has the same shapes (rwkv5.py:195, rwkv5_2.py:199).  The adapter hands
``log(w)`` as one ``(H,N)`` tensor to the WKV6 op (its ``w`` is the log decay; flag ``HIPRWKV_W_PER_HEAD``), so no
per-token decay is materialised; the decay cotangent comes back summed over batch and tokens.  With bf16 I/O ``log(w)`` is rounded
to bf16 once more (relative error of the decay 2^-9 |log w| per step).
"""
import torch

from . import ops


class HipRWKV:
    #: True -> returned state follows the associative-scan variants; False -> BaseRWKV (rwkv5.py:179)
    assoc_compat = True

    @classmethod
    def inner_loop(cls, r, k, v, w, time_first, s, length, new_starts):
        batched = r.dim() == 4
        if not batched:
            r, k, v, s = (x[None] for x in (r, k, v, s))
            if torch.is_tensor(new_starts) and new_starts.dim() == 1:
                new_starts = new_starts[None]
        B, T, H, N = r.shape
        logw = torch.log(w.float().reshape(H, -1)).expand(H, N).to(r.dtype).contiguous()   # HIPRWKV_W_PER_HEAD
        u = time_first.reshape(H, -1).expand(H, N).contiguous()
        new_s, y = ops.wkv6(r, k, v, logw, u, s, length, new_starts, cls.assoc_compat)
        new_s = new_s.to(r.dtype)
        if not batched:
            new_s, y = new_s[0], y[0]
        return new_s, y
