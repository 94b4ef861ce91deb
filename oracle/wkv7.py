"""Float64 NumPy oracle for the RWKV-7 WKV recurrence (checker only, never shipped).

Restates, without importing it, the algorithm of the reference:

* ``wkv7_base``            -- ``BaseRWKV.inner_loop``            /root/reference/src/jaxrwkv/rwkv7.py:200-220
* ``wkv7_assoc_literal``   -- ``AssociativeScanRWKV.inner_loop`` /root/reference/src/jaxrwkv/rwkv7.py:321-346
  (the parity oracle; its prefix scan is evaluated as a left fold of the same
  combine function, which equals the tree evaluation up to rounding)
* ``wkv7_assoc_scan``      -- the same operands pushed through a real log-depth
  (Hillis-Steele) scan with the combine of rwkv7.py:335-341; this is the form
  the CPU baseline times.
* ``wkv7_bwd``             -- analytic vector-Jacobian product of ``wkv7_base``
  (pinned in tests by central finite differences and by torch autograd of an
  independent restatement).

All functions take a leading batch axis, i.e. what the reference obtains with
``jax.vmap`` (rwkv7.py:419-431): r,w,k,v,a,b ``(B,T,H,N)``; s ``(B,H,N,N)`` with
``s[b,h,i,j]`` = value row i, key column j (rwkv7.py:216-218); length ``(B,)``;
new_starts ``(B,T)`` bool.  ``compat=True`` reproduces the two places where the
associative form differs from the sequential one:

Q1  ``out[t] = scan_s[t+1] @ r[t]`` (rwkv7.py:344) and element ``t+1`` of the
    scan is zeroed when ``new_starts[t+1]`` (rwkv7.py:331-333): y[t] is 0 there.
Q2  ``s = scan_s[length]`` (rwkv7.py:345) is the state *entering* position
    ``length``: zero if ``length < T`` and ``new_starts[length]``.
"""
import numpy as np


def _prep(r, w, k, v, a, b, s, length, new_starts):
    f = lambda x: np.asarray(x, dtype=np.float64)
    r, w, k, v, a, b, s = map(f, (r, w, k, v, a, b, s))
    B, T, H, N = r.shape
    if length is None:
        length = np.full((B,), T)          # llm.py:78-79
    if new_starts is None:
        new_starts = np.zeros((B, T), bool)  # llm.py:80-81
    length = np.minimum(np.broadcast_to(np.asarray(length, dtype=np.int64), (B,)), T)
    new_starts = np.broadcast_to(np.asarray(new_starts, dtype=bool), (B, T))
    return r, w, k, v, a, b, s, length, new_starts


def wkv7_base(r, w, k, v, a, b, s, length=None, new_starts=None, compat=False, return_sa=False):
    """Sequential recurrence, rwkv7.py:200-220.  Returns (out_s, y[, sa])."""
    r, w, k, v, a, b, s, length, new_starts = _prep(r, w, k, v, a, b, s, length, new_starts)
    B, T, H, N = r.shape
    d = np.exp(-np.exp(w))                                   # :201
    S = s.copy()
    out_s = s.copy()                                         # :203
    y = np.zeros_like(r)
    sa_all = np.zeros_like(r)
    for t in range(T):
        S = np.where(new_starts[:, t, None, None, None], 0.0, S)        # :207
        sa = np.einsum('bhij,bhj->bhi', S, a[:, t])                      # :216
        S = (S * d[:, t, :, None, :]
             + v[:, t, :, :, None] * k[:, t, :, None, :]
             + sa[..., None] * b[:, t, :, None, :])                     # :217
        y[:, t] = np.einsum('bhij,bhj->bhi', S, r[:, t])                 # :218
        sa_all[:, t] = sa
        out_s = np.where((t < length)[:, None, None, None], S, out_s)    # :219
    if compat:
        y, out_s = _apply_compat(y, out_s, s, length, new_starts)
    if return_sa:
        return out_s, y, sa_all
    return out_s, y


def _apply_compat(y, out_s, s, length, new_starts):
    B, T = new_starts.shape
    y = y.copy()
    out_s = out_s.copy()
    nxt = np.zeros((B, T), bool)
    nxt[:, :-1] = new_starts[:, 1:]
    y[nxt] = 0.0                                                          # Q1
    for bi in range(B):
        L = int(length[bi])
        if L < T and new_starts[bi, L]:
            out_s[bi] = 0.0                                               # Q2
        elif L == 0:
            out_s[bi] = s[bi]
    return y, out_s


def _assoc_operands(r, w, k, v, a, b, s, new_starts):
    """Scan operands of rwkv7.py:322-333 for one sequence: all_A, all_W (T+1,H,N,N)."""
    T, H, N = r.shape
    d = np.exp(-np.exp(w))                                                # :322
    W = np.einsum('thi,ij->thij', d, np.eye(N)) + a[..., :, None] * b[..., None, :]   # :324,327
    A = v[..., :, None] * k[..., None, :]                                 # :325,328
    all_A = np.concatenate((s[None], A))                                  # :329
    all_W = np.concatenate((np.zeros_like(W[:1]), W))                     # :330
    ns = np.concatenate((new_starts, np.zeros(1, bool)))[:, None, None, None]   # :331
    all_A = np.where(ns, 0.0, all_A)                                      # :332
    all_W = np.where(ns, 0.0, all_W)                                      # :333
    return all_A, all_W


def wkv7_assoc_literal(r, w, k, v, a, b, s, length=None, new_starts=None):
    """rwkv7.py:321-346 with the prefix scan evaluated as a left fold."""
    r, w, k, v, a, b, s, length, new_starts = _prep(r, w, k, v, a, b, s, length, new_starts)
    B, T, H, N = r.shape
    y = np.zeros_like(r)
    out_s = np.zeros_like(s)
    for bi in range(B):
        all_A, all_W = _assoc_operands(r[bi], w[bi], k[bi], v[bi], a[bi], b[bi], s[bi], new_starts[bi])
        scan_s = np.empty_like(all_A)
        scan_s[0] = all_A[0]
        for i in range(1, T + 1):
            scan_s[i] = all_A[i] + scan_s[i - 1] @ all_W[i]               # :339 (A12 = A2 + A1 @ W2)
        y[bi] = np.einsum('thij,thj->thi', scan_s[1:], r[bi])             # :344
        out_s[bi] = scan_s[int(length[bi])]                               # :345
    return out_s, y


def assoc_scan_1seq(all_A, all_W, dtype=np.float32):
    """Log-depth inclusive scan (Hillis-Steele) with the combine of rwkv7.py:335-341.

    Operates on one sequence; returns scan_s (T+1,H,N,N).  Used by the CPU
    baseline, where the work (2 N^3-matmuls per combine) is what is timed.
    """
    A = np.ascontiguousarray(all_A, dtype=dtype)
    W = np.ascontiguousarray(all_W, dtype=dtype)
    n = A.shape[0]
    off = 1
    while off < n:
        A1, W1 = A[:-off], W[:-off]
        A2, W2 = A[off:], W[off:]
        newA = A2 + np.matmul(A1, W2)
        newW = np.matmul(W1, W2)
        A = np.concatenate((A[:off], newA))
        W = np.concatenate((W[:off], newW))
        off *= 2
    return A


def wkv7_assoc_scan(r, w, k, v, a, b, s, length=None, new_starts=None, dtype=np.float32):
    """Same result as ``wkv7_assoc_literal`` but through the log-depth scan, in ``dtype``."""
    r, w, k, v, a, b, s, length, new_starts = _prep(r, w, k, v, a, b, s, length, new_starts)
    B, T, H, N = r.shape
    y = np.zeros(r.shape, dtype)
    out_s = np.zeros(s.shape, dtype)
    for bi in range(B):
        all_A, all_W = _assoc_operands(r[bi], w[bi], k[bi], v[bi], a[bi], b[bi], s[bi], new_starts[bi])
        scan_s = assoc_scan_1seq(all_A, all_W, dtype)
        y[bi] = np.einsum('thij,thj->thi', scan_s[1:], r[bi].astype(dtype))
        out_s[bi] = scan_s[int(length[bi])]
    return out_s, y


def wkv7_bwd(r, w, k, v, a, b, s, length, new_starts, dy, ds_out, compat=False):
    """Vector-Jacobian product of ``wkv7_base`` (and of its ``compat`` variant).

    dy ``(B,T,H,N)`` is the cotangent of y, ds_out ``(B,H,N,N)`` of the returned
    state.  Returns (dr, dw, dk, dv, da, db, ds).
    """
    r, w, k, v, a, b, s, length, new_starts = _prep(r, w, k, v, a, b, s, length, new_starts)
    dy = np.asarray(dy, np.float64).copy()
    ds_out = np.asarray(ds_out, np.float64).copy()
    B, T, H, N = r.shape
    d = np.exp(-np.exp(w))
    ds0_extra = np.zeros_like(s)
    if compat:
        nxt = np.zeros((B, T), bool)
        nxt[:, :-1] = new_starts[:, 1:]
        dy[nxt] = 0.0
    for bi in range(B):
        L = int(length[bi])
        if compat and L < T and new_starts[bi, L]:
            ds_out[bi] = 0.0
        if L == 0:
            ds0_extra[bi] = ds_out[bi]
            ds_out[bi] = 0.0
    # forward sweep storing the states entering every step
    Sp = np.zeros((T, B, H, N, N))
    S = s.copy()
    for t in range(T):
        S = np.where(new_starts[:, t, None, None, None], 0.0, S)
        Sp[t] = S
        sa = np.einsum('bhij,bhj->bhi', S, a[:, t])
        S = S * d[:, t, :, None, :] + v[:, t, :, :, None] * k[:, t, :, None, :] + sa[..., None] * b[:, t, :, None, :]
    dr, dw, dk, dv, da, db = (np.zeros_like(r) for _ in range(6))
    G = np.zeros_like(s)
    for t in range(T - 1, -1, -1):
        Sin = Sp[t]
        sa = np.einsum('bhij,bhj->bhi', Sin, a[:, t])
        St = Sin * d[:, t, :, None, :] + v[:, t, :, :, None] * k[:, t, :, None, :] + sa[..., None] * b[:, t, :, None, :]
        G = G + dy[:, t, :, :, None] * r[:, t, :, None, :]
        G = G + np.where((length - 1 == t)[:, None, None, None], ds_out, 0.0)
        dr[:, t] = np.einsum('bhij,bhi->bhj', St, dy[:, t])
        dv[:, t] = np.einsum('bhij,bhj->bhi', G, k[:, t])
        dk[:, t] = np.einsum('bhij,bhi->bhj', G, v[:, t])
        db[:, t] = np.einsum('bhij,bhi->bhj', G, sa)
        dsa = np.einsum('bhij,bhj->bhi', G, b[:, t])
        da[:, t] = np.einsum('bhij,bhi->bhj', Sin, dsa)
        dd = np.einsum('bhij,bhij->bhj', G, Sin)
        dw[:, t] = dd * d[:, t] * (-np.exp(w[:, t]))
        G = G * d[:, t, :, None, :] + dsa[..., None] * a[:, t, :, None, :]
        G = np.where(new_starts[:, t, None, None, None], 0.0, G)
    return dr, dw, dk, dv, da, db, G + ds0_extra
