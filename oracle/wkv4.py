"""Float64 NumPy oracle for the RWKV-4 WKV recurrence (checker only, never shipped).

* ``wkv4_base``           -- ``BaseRWKV.inner_loop``            /root/reference/src/jaxrwkv/rwkv4.py:144-172
* ``wkv4_assoc_literal``  -- ``AssociativeScanRWKV.inner_loop`` /root/reference/src/jaxrwkv/rwkv4.py:253-300
  (prefix scan evaluated as a left fold of ``a_scan_loop`` :266-284)
* ``wkv4_ffi``            -- the operand convention of the reference's native
  op (rwkv4.py:311-323, 403-406): ``w`` arrives as ``-exp(time_decay)`` and the
  receptance is applied by the caller.

Batched layout: r,k,v ``(B,T,C)``; time_decay, time_first ``(C,)``; s ``(B,3,C)`` =
(aa, bb, pp) with the reset value (0, 0, -1e30) (rwkv4.py:118-123, 149-150).
``compat=True``: returned state is the one *entering* position ``length``
(rwkv4.py:300), i.e. the reset value when ``length < T`` and ``new_starts[length]``.
"""
import numpy as np

RESET_PP = -1e30


def _prep(k, v, s, length, new_starts):
    k, v, s = (np.asarray(x, dtype=np.float64) for x in (k, v, s))
    B, T, C = k.shape
    if length is None:
        length = np.full((B,), T)
    if new_starts is None:
        new_starts = np.zeros((B, T), bool)
    length = np.minimum(np.broadcast_to(np.asarray(length, dtype=np.int64), (B,)), T)
    new_starts = np.broadcast_to(np.asarray(new_starts, dtype=bool), (B, T))
    return k, v, s, length, new_starts


def wkv4_ffi(w_neg, u, k, v, s, length=None, new_starts=None, compat=False):
    """Recurrence of rwkv4.py:147-171 with ``w_neg = -exp(time_decay)`` and no receptance.

    Returns (new_s (B,3,C), wkv (B,T,C)).
    """
    k, v, s, length, new_starts = _prep(k, v, s, length, new_starts)
    w = np.asarray(w_neg, np.float64)
    u = np.asarray(u, np.float64)
    B, T, C = k.shape
    aa, bb, pp = s[:, 0].copy(), s[:, 1].copy(), s[:, 2].copy()
    out_s = s.copy()
    y = np.zeros_like(k)
    for t in range(T):
        ns = new_starts[:, t, None]
        aa = np.where(ns, 0.0, aa)                                        # :153
        bb = np.where(ns, 0.0, bb)
        pp = np.where(ns, RESET_PP, pp)
        ww = u + k[:, t]                                                  # :156
        qq = np.maximum(pp, ww)
        e1 = np.exp(pp - qq)
        e2 = np.exp(ww - qq)
        y[:, t] = (e1 * aa + e2 * v[:, t]) / (e1 * bb + e2)               # :160-162
        ww = pp + w                                                       # :165
        qq = np.maximum(ww, k[:, t])
        e1 = np.exp(ww - qq)
        e2 = np.exp(k[:, t] - qq)
        aa = e1 * aa + e2 * v[:, t]                                       # :170
        bb = e1 * bb + e2
        pp = qq
        snap = (t < length)[:, None, None]
        out_s = np.where(snap, np.stack([aa, bb, pp], axis=1), out_s)     # :171
    if compat:
        out_s = out_s.copy()
        for bi in range(B):
            L = int(length[bi])
            if L < T and new_starts[bi, L]:
                out_s[bi, 0] = 0.0
                out_s[bi, 1] = 0.0
                out_s[bi, 2] = RESET_PP
    return out_s, y


def wkv4_base(r, k, v, time_decay, time_first, s, length=None, new_starts=None, compat=False):
    """``inner_loop`` signature of rwkv4.py:144: applies ``w=-exp(time_decay)`` (:145) and ``r*wkv`` (:163)."""
    out_s, y = wkv4_ffi(-np.exp(np.asarray(time_decay, np.float64)), time_first, k, v, s, length, new_starts, compat)
    return out_s, np.asarray(r, np.float64) * y


def wkv4_assoc_literal(r, k, v, time_decay, time_first, s, length=None, new_starts=None):
    """rwkv4.py:253-300 with the scan evaluated as a left fold of its combine."""
    k, v, s, length, new_starts = _prep(k, v, s, length, new_starts)
    r = np.asarray(r, np.float64)
    w = -np.exp(np.asarray(time_decay, np.float64))                       # :254
    u = np.asarray(time_first, np.float64)
    B, T, C = k.shape
    out = np.zeros_like(k)
    out_s = np.zeros_like(s)
    for bi in range(B):
        AA = np.concatenate((s[bi, 0:1], v[bi]))                          # :257
        BB = np.ones_like(AA)
        BB[0] = s[bi, 1]                                                  # :258-259
        PP = np.concatenate((s[bi, 2:3], k[bi]))                          # :260
        ns = np.concatenate((new_starts[bi], np.zeros(1, bool)))          # :262
        AA = np.where(ns[:, None], 0.0, AA)                               # :264-266
        BB = np.where(ns[:, None], 0.0, BB)
        PP = np.where(ns[:, None], RESET_PP, PP)
        sA, sB, sP = np.empty_like(AA), np.empty_like(BB), np.empty_like(PP)
        sA[0], sB[0], sP[0] = AA[0], BB[0], PP[0]
        for i in range(1, T + 1):
            if ns[i]:                                                     # where(r2, x2, xN) :279-283
                sA[i], sB[i], sP[i] = AA[i], BB[i], PP[i]
                continue
            ww = sP[i - 1] + 1 * w                                        # d = E2 - E1 = 1 in a left fold (:271-273)
            qq = np.maximum(ww, PP[i])
            sA[i] = sA[i - 1] * np.exp(ww - qq) + AA[i] * np.exp(PP[i] - qq)   # :275
            sB[i] = sB[i - 1] * np.exp(ww - qq) + BB[i] * np.exp(PP[i] - qq)   # :276
            sP[i] = qq
        aa, bb, pp = sA[:T], sB[:T], sP[:T]                               # :288-290
        ww = u[None] + k[bi]                                              # :292
        qq = np.maximum(pp, ww)
        e1 = np.exp(pp - qq)
        e2 = np.exp(ww - qq)
        out[bi] = r[bi] * ((e1 * aa + e2 * v[bi]) / (e1 * bb + e2))        # :295-298
        L = int(length[bi])
        out_s[bi] = np.stack([sA[L], sB[L], sP[L]])                        # :300
    return out_s, out


def wkv4_ffi_bwd(w_neg, u, k, v, s, length, new_starts, gy, gs_new, compat=False):
    """Reverse-mode derivative of ``wkv4_ffi`` step by step through the max-tracked recurrence (the program of
    rwkv4.py:147-171, so that it agrees with autodiff of the reference's ScanRWKV): cotangents gy of the
    un-gated output and gs_new of the returned raw state (aa, bb, pp).

    Returns (gw (B,C), gu (B,C), gk, gv, gs (B,3,C)); gw and gu are per sequence, to be summed over B by the
    caller as the reference does (rwkv4.py:351).  ``max`` passes its cotangent to the larger argument.
    """
    k, v, s, length, new_starts = _prep(k, v, s, length, new_starts)
    w = np.asarray(w_neg, np.float64)
    u = np.asarray(u, np.float64)
    gy = np.asarray(gy, np.float64)
    gs_new = np.asarray(gs_new, np.float64).copy()
    B, T, C = k.shape
    gs_extra = np.zeros_like(s)
    for bi in range(B):
        L = int(length[bi])
        if compat and L < T and new_starts[bi, L]:
            gs_new[bi] = 0.0
        if L == 0:
            gs_extra[bi] = gs_new[bi]
            gs_new[bi] = 0.0
    # forward sweep keeping the state entering every step
    st = np.zeros((T, B, 3, C))
    aa, bb, pp = s[:, 0].copy(), s[:, 1].copy(), s[:, 2].copy()
    for t in range(T):
        ns = new_starts[:, t, None]
        aa, bb, pp = np.where(ns, 0.0, aa), np.where(ns, 0.0, bb), np.where(ns, RESET_PP, pp)
        st[t, :, 0], st[t, :, 1], st[t, :, 2] = aa, bb, pp
        ww = pp + w
        qq = np.maximum(ww, k[:, t])
        f1, f2 = np.exp(ww - qq), np.exp(k[:, t] - qq)
        aa, bb, pp = f1 * aa + f2 * v[:, t], f1 * bb + f2, qq
    gk, gv = np.zeros_like(k), np.zeros_like(v)
    gw, gu = np.zeros((B, C)), np.zeros((B, C))
    g_aa, g_bb, g_pp = np.zeros((B, C)), np.zeros((B, C)), np.zeros((B, C))
    for t in range(T - 1, -1, -1):
        inj = (length - 1 == t)[:, None]
        g_aa = g_aa + np.where(inj, gs_new[:, 0], 0.0)
        g_bb = g_bb + np.where(inj, gs_new[:, 1], 0.0)
        g_pp = g_pp + np.where(inj, gs_new[:, 2], 0.0)
        aa, bb, pp = st[t, :, 0], st[t, :, 1], st[t, :, 2]
        kt, vt = k[:, t], v[:, t]
        # state update
        ww2 = pp + w
        q2 = np.maximum(ww2, kt)
        f1, f2 = np.exp(ww2 - q2), np.exp(kt - q2)
        g_f1 = g_aa * aa + g_bb * bb
        g_f2 = g_aa * vt + g_bb
        n_aa, n_bb = g_aa * f1, g_bb * f1
        g_v = g_aa * f2
        g_q2 = g_pp - g_f1 * f1 - g_f2 * f2
        g_ww2 = g_f1 * f1 + np.where(ww2 >= kt, g_q2, 0.0)
        g_k = g_f2 * f2 + np.where(ww2 >= kt, 0.0, g_q2)
        n_pp = g_ww2
        gw += g_ww2
        # output
        ww = u + kt
        q = np.maximum(pp, ww)
        e1, e2 = np.exp(pp - q), np.exp(ww - q)
        A, Bd = e1 * aa + e2 * vt, e1 * bb + e2
        g_A = gy[:, t] / Bd
        g_B = -gy[:, t] * A / (Bd * Bd)
        g_e1 = g_A * aa + g_B * bb
        g_e2 = g_A * vt + g_B
        n_aa += g_A * e1
        n_bb += g_B * e1
        g_v += g_A * e2
        g_q = -g_e1 * e1 - g_e2 * e2
        n_pp += g_e1 * e1 + np.where(pp >= ww, g_q, 0.0)
        g_ww = g_e2 * e2 + np.where(pp >= ww, 0.0, g_q)
        gu += g_ww
        g_k += g_ww
        gk[:, t], gv[:, t] = g_k, g_v
        ns = new_starts[:, t, None]
        g_aa, g_bb, g_pp = np.where(ns, 0.0, n_aa), np.where(ns, 0.0, n_bb), np.where(ns, 0.0, n_pp)
    gs = np.stack([g_aa, g_bb, g_pp], axis=1) + gs_extra
    return gw, gu, gk, gv, gs
