"""Pins the RWKV-5 oracle: closed form of the constant-decay recurrence and agreement with the WKV6 oracle."""
import numpy as np
import pytest

from oracle import wkv5 as o5
from oracle import wkv6 as o6


def inputs(B, T, H, N, seed, per_channel):
    g = np.random.default_rng(seed)
    r, k, v = (g.standard_normal((B, T, H, N)) for _ in range(3))
    w = np.exp(-np.exp(g.standard_normal((H, N if per_channel else 1, 1)) - 1.0))
    u = np.exp(0.3 * g.standard_normal((H, N if per_channel else 1, 1)))
    s = 0.1 * g.standard_normal((B, H, N, N))
    return r, k, v, w, u, s


@pytest.mark.parametrize("per_channel", [False, True])
def test_closed_form(per_channel):
    """y_t = r_t.(u (.) k_t) v_t + sum_{s<t} (r_t . w^(t-1-s) . k_s) v_s + (r_t . w^t) S0."""
    B, T, H, N = 1, 7, 2, 8
    r, k, v, w, u, s = inputs(B, T, H, N, 0, per_channel)
    _, y = o5.wkv5_base(r, k, v, w, u, s)
    wv = np.broadcast_to(w.reshape(H, -1), (H, N))
    uv = np.broadcast_to(u.reshape(H, -1), (H, N))
    for t in range(T):
        ref = np.einsum('hi,hi,hj->hj', r[0, t] * uv, k[0, t], v[0, t])
        ref += np.einsum('hi,hij->hj', r[0, t] * wv ** t, s[0])
        for q in range(t):
            ref += np.einsum('hi,hi,hj->hj', r[0, t] * wv ** (t - 1 - q), k[0, q], v[0, q])
        np.testing.assert_allclose(y[0, t], ref, rtol=1e-11, atol=1e-12)


@pytest.mark.parametrize("per_channel", [False, True])
@pytest.mark.parametrize("compat", [False, True])
def test_equals_wkv6_with_log_decay(per_channel, compat):
    B, T, H, N = 2, 19, 2, 8
    r, k, v, w, u, s = inputs(B, T, H, N, 1, per_channel)
    g = np.random.default_rng(2)
    ns = g.random((B, T)) < 0.15
    length = np.array([11, 19])
    ns[0, 11] = True
    s5, y5 = o5.wkv5_base(r, k, v, w, u, s, length, ns, compat=compat)
    logw = np.broadcast_to(np.log(np.broadcast_to(w.reshape(H, -1), (H, N)))[None, None], (B, T, H, N))
    s6, y6 = o6.wkv6_base(r, k, v, logw, np.broadcast_to(u.reshape(H, -1), (H, N)), s, length, ns, compat=compat)
    np.testing.assert_allclose(y5, y6, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(s5, s6, rtol=1e-11, atol=1e-12)
