"""Float64 NumPy oracle for the RWKV-6 WKV recurrence (checker only, never shipped).

* ``wkv6_base``           -- ``BaseRWKV.inner_loop``            /root/reference/src/jaxrwkv/rwkv6.py:175-191
* ``wkv6_assoc_literal``  -- ``AssociativeScanRWKV.inner_loop`` /root/reference/src/jaxrwkv/rwkv6.py:278-302
  (prefix scan evaluated as a left fold of the same combine, reset flag included)
* ``wkv6_bwd``            -- analytic vector-Jacobian product of ``wkv6_base``.

Batched layout: r,k,v,w ``(B,T,H,N)`` (the reference's trailing singleton of
``w``, rwkv6.py:217, is dropped), ``w`` is the *log* decay ``-exp(raw)``
(rwkv6.py:218), u = ``time_faaaa`` ``(H,N)``; s ``(B,H,N,N)`` with ``s[b,h,i,j]`` =
key row i, value column j (rwkv6.py:187-189).  ``compat=True`` applies the one
divergence of the associative form: the returned state is ``scan_s[length]``
(rwkv6.py:301), i.e. zero when ``length < T`` and ``new_starts[length]``.
The outputs of the two forms agree (rwkv6.py:300 reads ``scan_s[:-1]``).
"""
import numpy as np


def _prep(r, k, v, w, u, s, length, new_starts):
    f = lambda x: np.asarray(x, dtype=np.float64)
    r, k, v, w, u, s = map(f, (r, k, v, w, u, s))
    B, T, H, N = r.shape
    w = w.reshape(B, T, H, N)
    u = u.reshape(H, N)
    if length is None:
        length = np.full((B,), T)
    if new_starts is None:
        new_starts = np.zeros((B, T), bool)
    length = np.minimum(np.broadcast_to(np.asarray(length, dtype=np.int64), (B,)), T)
    new_starts = np.broadcast_to(np.asarray(new_starts, dtype=bool), (B, T))
    return r, k, v, w, u, s, length, new_starts


def wkv6_base(r, k, v, w, u, s, length=None, new_starts=None, compat=False):
    """Sequential recurrence, rwkv6.py:175-191.  Returns (out_s, y)."""
    r, k, v, w, u, s, length, new_starts = _prep(r, k, v, w, u, s, length, new_starts)
    B, T, H, N = r.shape
    dec = np.exp(w)                                                       # :176
    S = s.copy()
    out_s = s.copy()
    y = np.zeros_like(r)
    for t in range(T):
        S = np.where(new_starts[:, t, None, None, None], 0.0, S)          # :182
        A = k[:, t, :, :, None] * v[:, t, :, None, :]                     # :187
        y[:, t] = np.einsum('bhi,bhij->bhj', r[:, t], u[None, :, :, None] * A + S)   # :188
        S = A + dec[:, t, :, :, None] * S                                 # :189
        out_s = np.where((t < length)[:, None, None, None], S, out_s)     # :190
    if compat:
        out_s = out_s.copy()
        for bi in range(B):
            L = int(length[bi])
            if L < T and new_starts[bi, L]:
                out_s[bi] = 0.0
    return out_s, y


def wkv6_assoc_literal(r, k, v, w, u, s, length=None, new_starts=None):
    """rwkv6.py:278-302 with the scan as a left fold of ``a_scan_loop`` (:292-298)."""
    r, k, v, w, u, s, length, new_starts = _prep(r, k, v, w, u, s, length, new_starts)
    B, T, H, N = r.shape
    dec = np.exp(w)                                                       # :279
    y = np.zeros_like(r)
    out_s = np.zeros_like(s)
    for bi in range(B):
        A = k[bi][..., :, None] * v[bi][..., None, :]                     # :284
        all_A = np.concatenate((s[bi][None], A))                          # :285
        all_W = np.concatenate((np.zeros_like(dec[bi][:1]), dec[bi]))[..., None]   # :286
        ns = np.concatenate((new_starts[bi], np.zeros(1, bool)))          # :287
        all_A = np.where(ns[:, None, None, None], 0.0, all_A)             # :289
        all_W = np.where(ns[:, None, None, None], 0.0, all_W)             # :290
        scan_s = np.empty_like(all_A)
        scan_s[0] = all_A[0]
        for i in range(1, T + 1):
            if ns[i]:                                                     # where(r2, A2, A12) :298
                scan_s[i] = all_A[i]
            else:
                scan_s[i] = all_A[i] + all_W[i] * scan_s[i - 1]           # :296
        y[bi] = np.einsum('thi,thij->thj', r[bi], u[None, :, :, None] * A + scan_s[:-1])   # :300
        out_s[bi] = scan_s[int(length[bi])]                               # :301
    return out_s, y


def wkv6_bwd(r, k, v, w, u, s, length, new_starts, dy, ds_out, compat=False):
    """Vector-Jacobian product of ``wkv6_base``.  Returns (dr, dk, dv, dw, du, ds)."""
    r, k, v, w, u, s, length, new_starts = _prep(r, k, v, w, u, s, length, new_starts)
    dy = np.asarray(dy, np.float64)
    ds_out = np.asarray(ds_out, np.float64).copy()
    B, T, H, N = r.shape
    dec = np.exp(w)
    ds0_extra = np.zeros_like(s)
    for bi in range(B):
        L = int(length[bi])
        if compat and L < T and new_starts[bi, L]:
            ds_out[bi] = 0.0
        if L == 0:
            ds0_extra[bi] = ds_out[bi]
            ds_out[bi] = 0.0
    Sp = np.zeros((T, B, H, N, N))
    S = s.copy()
    for t in range(T):
        S = np.where(new_starts[:, t, None, None, None], 0.0, S)
        Sp[t] = S
        S = k[:, t, :, :, None] * v[:, t, :, None, :] + dec[:, t, :, :, None] * S
    dr, dk, dv, dw = (np.zeros_like(r) for _ in range(4))
    du = np.zeros_like(u)
    G = np.zeros_like(s)
    for t in range(T - 1, -1, -1):
        Sin = Sp[t]
        G = G + np.where((length - 1 == t)[:, None, None, None], ds_out, 0.0)   # grad wrt S_t
        A = k[:, t, :, :, None] * v[:, t, :, None, :]
        GA = G + (r[:, t] * u[None])[..., :, None] * dy[:, t, :, None, :]        # grad wrt A_t
        dk[:, t] = np.einsum('bhij,bhj->bhi', GA, v[:, t])
        dv[:, t] = np.einsum('bhij,bhi->bhj', GA, k[:, t])
        dr[:, t] = np.einsum('bhij,bhj->bhi', u[None, :, :, None] * A + Sin, dy[:, t])
        du += np.einsum('bhi,bhij,bhj->hi', r[:, t], A, dy[:, t])
        dw[:, t] = np.einsum('bhij,bhij->bhi', G, Sin) * dec[:, t]
        G = dec[:, t, :, :, None] * G + r[:, t, :, :, None] * dy[:, t, :, None, :]
        G = np.where(new_starts[:, t, None, None, None], 0.0, G)
    return dr, dk, dv, dw, du, G + ds0_extra
