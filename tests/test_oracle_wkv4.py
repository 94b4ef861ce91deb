"""Pins the WKV4 oracle: log-sum-exp closed form, pp closed form, associative restatement, invariants."""
import numpy as np
import pytest
from scipy.special import logsumexp

from oracle import wkv4 as o4
from tests.inputs import wkv4_inputs


def test_closed_form_softmax_average_and_pp():
    x = wkv4_inputs(2, 14, 6, seed=0, default_state=False)
    k, v, w, u, s = x["k"], x["v"], x["w"], x["u"], x["s"]
    out_s, y = o4.wkv4_ffi(w, u, k, v, s)
    B, T, C = k.shape
    aa0, bb0, pp0 = s[:, 0], s[:, 1], s[:, 2]
    for t in range(T):
        # log-weights of: the carried state, past tokens s<t, the current token with the bonus u
        logs = [pp0 + t * w] + [k[:, q] + (t - 1 - q) * w for q in range(t)] + [u + k[:, t]]
        lw = np.stack(logs)
        num_vals = np.stack([aa0] + [v[:, q] for q in range(t)] + [v[:, t]])
        den_vals = np.stack([bb0] + [np.ones_like(aa0)] * (t + 1))
        m = lw.max(0)
        num = np.sum(np.exp(lw - m) * num_vals, 0)
        den = np.sum(np.exp(lw - m) * den_vals, 0)
        np.testing.assert_allclose(y[:, t], num / den, rtol=1e-12, atol=1e-13)
    # final state: pp_T = max(pp0 + T w, max_s k_s + (T-1-s) w); (aa/bb, log bb + pp) representation-free
    lw = np.stack([pp0 + T * w] + [k[:, q] + (T - 1 - q) * w for q in range(T)])
    np.testing.assert_allclose(out_s[:, 2], lw.max(0), rtol=1e-13, atol=0)
    den_vals = np.stack([bb0] + [np.ones_like(aa0)] * T)
    np.testing.assert_allclose(np.log(out_s[:, 1]) + out_s[:, 2], logsumexp(lw, axis=0, b=den_vals), rtol=1e-12, atol=1e-12)


def test_default_state_first_token_is_v():
    x = wkv4_inputs(2, 3, 5, seed=1)
    _, y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"])
    np.testing.assert_allclose(y[:, 0], x["v"][:, 0], rtol=1e-14)


@pytest.mark.parametrize("seed", [0, 1])
def test_base_compat_equals_assoc_literal(seed):
    x = wkv4_inputs(3, 17, 5, seed=seed, p_reset=0.2, default_state=False, min_len=1)
    x["new_starts"][0, 0] = True
    x["length"][0] = 8
    x["new_starts"][0, 8] = True
    g = np.random.default_rng(seed)
    r = g.random(x["k"].shape)
    td = np.log(-x["w"])
    s1, y1 = o4.wkv4_base(r, x["k"], x["v"], td, x["u"], x["s"], x["length"], x["new_starts"], compat=True)
    s2, y2 = o4.wkv4_assoc_literal(r, x["k"], x["v"], td, x["u"], x["s"], x["length"], x["new_starts"])
    np.testing.assert_allclose(y1, y2, rtol=1e-12, atol=1e-13)
    np.testing.assert_allclose(s1, s2, rtol=1e-12, atol=1e-13)
    s3, _ = o4.wkv4_base(r, x["k"], x["v"], td, x["u"], x["s"], x["length"], x["new_starts"], compat=False)
    assert np.all(s2[0, 2] == o4.RESET_PP) and np.all(s3[0, 2] != o4.RESET_PP)


def test_split_carry_and_reset():
    x = wkv4_inputs(2, 20, 4, seed=2, default_state=False)
    k, v, w, u, s = x["k"], x["v"], x["w"], x["u"], x["s"]
    fs, fy = o4.wkv4_ffi(w, u, k, v, s)
    cut = 9
    sa, ya = o4.wkv4_ffi(w, u, k[:, :cut], v[:, :cut], s)
    sb, yb = o4.wkv4_ffi(w, u, k[:, cut:], v[:, cut:], sa)
    np.testing.assert_allclose(np.concatenate([ya, yb], 1), fy, rtol=1e-13, atol=0)
    np.testing.assert_allclose(sb, fs, rtol=1e-13, atol=0)
    sl, _ = o4.wkv4_ffi(w, u, k, v, s, length=np.array([cut, cut]))
    np.testing.assert_allclose(sl, sa, atol=0)
    ns = np.zeros((2, 20), bool)
    ns[:, cut] = True
    reset = np.zeros_like(s)
    reset[:, 2] = o4.RESET_PP
    sr, yr = o4.wkv4_ffi(w, u, k, v, s, None, ns)
    sz, yz = o4.wkv4_ffi(w, u, k[:, cut:], v[:, cut:], reset)
    np.testing.assert_allclose(yr[:, cut:], yz, rtol=1e-13, atol=0)
    np.testing.assert_allclose(sr, sz, rtol=1e-13, atol=0)


def test_large_k_is_stable():
    # the max-tracked form must not overflow where exp(k) would
    x = wkv4_inputs(1, 8, 3, seed=3)
    k = x["k"] * 300.0
    _, y = o4.wkv4_ffi(x["w"], x["u"], k, x["v"], x["s"])
    assert np.all(np.isfinite(y))
    assert np.all(np.abs(y) <= np.abs(x["v"]).max() + 1e-9)      # a convex combination of the v's


def _loss4(x, gy, gs, compat, **over):
    q = dict(x)
    q.update(over)
    out_s, y = o4.wkv4_ffi(q["w"], q["u"], q["k"], q["v"], q["s"], q["length"], q["new_starts"], compat=compat)
    out_s = np.where(out_s <= -1e29, 0.0, out_s)      # the constant "minus infinity" of a reset state would swamp the sum
    return np.sum(y * gy) + np.sum(out_s * gs)


@pytest.mark.parametrize("compat", [False, True])
@pytest.mark.parametrize("case", ["plain", "len_at_reset", "len0"])
def test_bwd_matches_finite_differences(compat, case):
    x = wkv4_inputs(2, 9, 5, seed=11, p_reset=0.25, default_state=False, min_len=2)
    x["new_starts"][0, 4] = True
    if case == "len_at_reset":
        x["length"][0] = 4
    if case == "len0":
        x["length"][:] = 0
    g = np.random.default_rng(5)
    gy, gs = g.standard_normal(x["k"].shape), g.standard_normal(x["s"].shape)
    gw, gu, gk, gv, gsi = o4.wkv4_ffi_bwd(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], gy, gs, compat=compat)
    grads = dict(w=gw.sum(0), u=gu.sum(0), k=gk, v=gv, s=gsi)
    eps = 1e-6
    for name, an in grads.items():
        for _ in range(12):
            idx = tuple(g.integers(0, n) for n in x[name].shape)
            xp, xm = x[name].copy(), x[name].copy()
            xp[idx] += eps
            xm[idx] -= eps
            fd = (_loss4(x, gy, gs, compat, **{name: xp}) - _loss4(x, gy, gs, compat, **{name: xm})) / (2 * eps)
            assert abs(fd - an[idx]) < 2e-6 * max(1.0, abs(fd)), (name, idx, fd, an[idx])


def test_bwd_matches_torch_autograd():
    import torch
    x = wkv4_inputs(2, 11, 6, seed=12, p_reset=0.2, default_state=False, min_len=3)
    g = np.random.default_rng(6)
    gy, gs = g.standard_normal(x["k"].shape), g.standard_normal(x["s"].shape)
    tt = {n: torch.tensor(x[n], dtype=torch.float64, requires_grad=True) for n in ("w", "u", "k", "v", "s")}
    ns, L = torch.tensor(x["new_starts"]), torch.tensor(x["length"])
    aa, bb, pp = tt["s"][:, 0], tt["s"][:, 1], tt["s"][:, 2]
    out_s, ys = tt["s"], []
    for t in range(11):
        keep = (~ns[:, t]).double()[:, None]
        aa, bb, pp = aa * keep, bb * keep, pp * keep + (1 - keep) * o4.RESET_PP
        kt, vt = tt["k"][:, t], tt["v"][:, t]
        # written with logaddexp-style primitives rather than the oracle's explicit e1/e2
        ww = tt["u"] + kt
        q = torch.maximum(pp, ww)
        ys.append((torch.exp(pp - q) * aa + torch.exp(ww - q) * vt) / (torch.exp(pp - q) * bb + torch.exp(ww - q)))
        ww2 = pp + tt["w"]
        q2 = torch.maximum(ww2, kt)
        aa, bb, pp = torch.exp(ww2 - q2) * aa + torch.exp(kt - q2) * vt, torch.exp(ww2 - q2) * bb + torch.exp(kt - q2), q2
        snap = (t < L).double()[:, None, None]
        out_s = snap * torch.stack([aa, bb, pp], 1) + (1 - snap) * out_s
    y = torch.stack(ys, 1)
    ((y * torch.tensor(gy)).sum() + (out_s * torch.tensor(gs)).sum()).backward()
    gw, gu, gk, gv, gsi = o4.wkv4_ffi_bwd(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], gy, gs)
    for name, an in (("w", gw.sum(0)), ("u", gu.sum(0)), ("k", gk), ("v", gv), ("s", gsi)):
        np.testing.assert_allclose(tt[name].grad.numpy(), an, rtol=1e-9, atol=1e-10, err_msg=name)
