"""Pins the WKV6 oracle: closed forms, the associative restatement, finite differences, torch autograd."""
import numpy as np
import pytest
import torch

from oracle import wkv6 as o6
from tests.inputs import wkv6_inputs


def _small(B=2, T=12, H=2, N=8, seed=0, **kw):
    kw.setdefault("p_reset", 0.2)
    return wkv6_inputs(B, T, H, N, seed=seed, **kw)


def test_no_bonus_unit_decay_is_exclusive_prefix_linear_attention():
    x = _small(resets=False, lengths=False, zero_state=True)
    u = np.zeros_like(x["u"])
    w = np.zeros_like(x["w"])                     # log-decay 0 -> decay 1
    out_s, y = o6.wkv6_base(x["r"], x["k"], x["v"], w, u, x["s"])
    kv = np.einsum('bthi,bthj->bthij', x["k"], x["v"])
    S_incl = np.cumsum(kv, axis=1)
    S_excl = S_incl - kv
    np.testing.assert_allclose(y, np.einsum('bthi,bthij->bthj', x["r"], S_excl), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(out_s, S_incl[:, -1], rtol=1e-12, atol=1e-12)


def test_general_closed_form_by_double_sum():
    x = _small(seed=1, T=9, resets=False, lengths=False)
    out_s, y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"])
    B, T, H, N = x["r"].shape
    Lc = np.cumsum(x["w"], axis=1)
    y_ref = np.zeros_like(y)
    for t in range(T):
        Le_t = Lc[:, t] - x["w"][:, t]            # exclusive cumulative log decay
        y_ref[:, t] += np.einsum('bhi,bhij->bhj', x["r"][:, t] * np.exp(Le_t), x["s"])
        y_ref[:, t] += np.sum(x["r"][:, t] * x["u"][None] * x["k"][:, t], -1, keepdims=True) * x["v"][:, t]
        for s in range(t):
            coef = np.sum(x["r"][:, t] * x["k"][:, s] * np.exp(Le_t - Lc[:, s]), -1, keepdims=True)
            y_ref[:, t] += coef * x["v"][:, s]
    np.testing.assert_allclose(y, y_ref, rtol=1e-11, atol=1e-12)


def test_constant_per_head_decay_is_rwkv5_form():
    # rwkv5.py:162-177 is the same recurrence with a decay that does not depend on t
    x = _small(seed=2, resets=False, lengths=False)
    w_head = x["w"][:1, :1]
    w = np.broadcast_to(w_head, x["w"].shape)
    out_s, y = o6.wkv6_base(x["r"], x["k"], x["v"], w, x["u"], x["s"])
    S = x["s"].copy()
    dec = np.exp(w_head[0, 0])[None, :, :, None]
    for t in range(x["r"].shape[1]):
        A = x["k"][:, t, :, :, None] * x["v"][:, t, :, None, :]
        np.testing.assert_allclose(y[:, t], np.einsum('bhi,bhij->bhj', x["r"][:, t], x["u"][None, :, :, None] * A + S), rtol=1e-12, atol=1e-12)
        S = A + dec * S
    np.testing.assert_allclose(out_s, S, rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_base_compat_equals_assoc_literal(seed):
    x = _small(seed=seed, T=16, p_reset=0.25)
    x["new_starts"][0, 0] = True
    x["length"][0] = 9
    x["new_starts"][0, 9] = True
    args = (x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"])
    s1, y1 = o6.wkv6_base(*args, compat=True)
    s2, y2 = o6.wkv6_assoc_literal(*args)
    np.testing.assert_allclose(y1, y2, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(s1, s2, rtol=1e-12, atol=1e-12)
    s3, y3 = o6.wkv6_base(*args, compat=False)
    np.testing.assert_allclose(y3, y2, rtol=1e-12, atol=1e-12)     # outputs agree in both conventions
    assert np.all(s2[0] == 0) and np.any(s3[0] != 0)


def test_split_carry_reset_and_length():
    x = _small(seed=3, T=18, resets=False, lengths=False)
    names = ("r", "k", "v", "w")
    full_s, full_y = o6.wkv6_base(*[x[n] for n in names], x["u"], x["s"])
    cut = 7
    s_a, y_a = o6.wkv6_base(*[x[n][:, :cut] for n in names], x["u"], x["s"])
    s_b, y_b = o6.wkv6_base(*[x[n][:, cut:] for n in names], x["u"], s_a)
    np.testing.assert_allclose(np.concatenate([y_a, y_b], 1), full_y, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(s_b, full_s, rtol=1e-12, atol=1e-12)
    s_len, _ = o6.wkv6_base(*[x[n] for n in names], x["u"], x["s"], length=np.array([cut, cut]))
    np.testing.assert_allclose(s_len, s_a, atol=0)
    ns = np.zeros((2, 18), bool)
    ns[:, cut] = True
    s_r, y_r = o6.wkv6_base(*[x[n] for n in names], x["u"], x["s"], None, ns)
    s_z, y_z = o6.wkv6_base(*[x[n][:, cut:] for n in names], x["u"], np.zeros_like(x["s"]))
    np.testing.assert_allclose(y_r[:, cut:], y_z, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(s_r, s_z, rtol=1e-12, atol=1e-12)


def _loss(x, compat, **over):
    q = dict(x)
    q.update(over)
    out_s, y = o6.wkv6_base(q["r"], q["k"], q["v"], q["w"], q["u"], q["s"], q["length"], q["new_starts"], compat=compat)
    return np.sum(y * q["dy"]) + np.sum(out_s * q["ds"])


@pytest.mark.parametrize("compat", [False, True])
@pytest.mark.parametrize("case", ["plain", "len_at_reset", "len0"])
def test_bwd_matches_finite_differences(compat, case):
    x = wkv6_inputs(2, 7, 2, 4, seed=11, p_reset=0.3)
    x["new_starts"][0, 3] = True
    if case == "len_at_reset":
        x["length"][0] = 3
    if case == "len0":
        x["length"][:] = 0
    grads = o6.wkv6_bwd(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"], compat=compat)
    g = np.random.default_rng(0)
    eps = 1e-6
    for name, an in zip(("r", "k", "v", "w", "u", "s"), grads):
        for _ in range(12):
            idx = tuple(g.integers(0, n) for n in x[name].shape)
            xp, xm = x[name].copy(), x[name].copy()
            xp[idx] += eps
            xm[idx] -= eps
            fd = (_loss(x, compat, **{name: xp}) - _loss(x, compat, **{name: xm})) / (2 * eps)
            assert abs(fd - an[idx]) < 1e-6 * max(1.0, abs(fd)), (name, idx, fd, an[idx])


def test_bwd_matches_torch_autograd():
    x = wkv6_inputs(2, 10, 2, 8, seed=12, p_reset=0.2)
    tt = {n: torch.tensor(x[n], dtype=torch.float64, requires_grad=True) for n in ("r", "k", "v", "w", "u", "s")}
    S, out_s, ys = tt["s"], tt["s"], []
    ns = torch.tensor(x["new_starts"])
    L = torch.tensor(x["length"])
    for t in range(10):
        S = S * (~ns[:, t]).double()[:, None, None, None]
        ru = tt["r"][:, t] * tt["u"][None]
        # y = (r.u.k) v + r^T S  -- written in the factored form, unlike the oracle
        ys.append((ru * tt["k"][:, t]).sum(-1, keepdim=True) * tt["v"][:, t] + torch.einsum('bhi,bhij->bhj', tt["r"][:, t], S))
        S = torch.exp(tt["w"][:, t])[..., None] * S + tt["k"][:, t, :, :, None] * tt["v"][:, t, :, None, :]
        snap = (t < L).double()[:, None, None, None]
        out_s = snap * S + (1 - snap) * out_s
    y = torch.stack(ys, 1)
    ((y * torch.tensor(x["dy"])).sum() + (out_s * torch.tensor(x["ds"])).sum()).backward()
    grads = o6.wkv6_bwd(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"])
    for name, an in zip(("r", "k", "v", "w", "u", "s"), grads):
        np.testing.assert_allclose(tt[name].grad.numpy(), an, rtol=1e-9, atol=1e-10, err_msg=name)
