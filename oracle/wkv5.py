"""Float64 NumPy oracle for the RWKV-5 / RWKV-5.2 recurrence (checker only, never shipped).

``wkv5_base`` restates ``BaseRWKV.inner_loop`` of /root/reference/src/jaxrwkv/rwkv5.py:162-181 (identical in
rwkv5_2.py:164-183): ``w`` is the decay itself, constant over the tokens, ``(H,1,1)`` or ``(H,N,1)``;
``time_first`` likewise; s ``(B,H,N,N)`` [key row, value column].  ``compat=True`` returns the state entering
position ``length`` as the associative-scan variants do (zero when ``length < T`` and ``new_starts[length]``).
Pinned by tests/test_oracle_wkv5.py against closed forms and against the WKV6 oracle with ``log w``.
"""
import numpy as np


def wkv5_base(r, k, v, w, time_first, s, length=None, new_starts=None, compat=False):
    r, k, v, s = (np.asarray(x, np.float64) for x in (r, k, v, s))
    B, T, H, N = r.shape
    w = np.broadcast_to(np.asarray(w, np.float64).reshape(H, -1, 1), (H, N, 1))
    u = np.broadcast_to(np.asarray(time_first, np.float64).reshape(H, -1, 1), (H, N, 1))
    length = np.full((B,), T) if length is None else np.minimum(np.broadcast_to(np.asarray(length, np.int64), (B,)), T)
    new_starts = np.zeros((B, T), bool) if new_starts is None else np.broadcast_to(np.asarray(new_starts, bool), (B, T))
    S = s.copy()
    out_s = s.copy()
    out = np.zeros_like(r)
    for t in range(T):
        S = np.where(new_starts[:, t, None, None, None], 0.0, S)          # :168
        at = k[:, t, :, :, None] * v[:, t, :, None, :]                    # :170-173
        out[:, t] = np.einsum('bhi,bhij->bhj', r[:, t], u[None] * at + S)  # :174
        S = at + w[None] * S                                              # :175
        out_s = np.where((t < length)[:, None, None, None], S, out_s)     # :176
    if compat:
        out_s = out_s.copy()
        for bi in range(B):
            L = int(length[bi])
            if L < T and new_starts[bi, L]:
                out_s[bi] = 0.0
    return out_s, out
