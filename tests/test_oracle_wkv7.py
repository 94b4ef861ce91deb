"""Pins the WKV7 oracle with closed forms, invariants, finite differences and torch autograd.

None of these checks retypes the oracle's recurrence: each one is a case where
mathematics fixes the answer by another route (a triangular-masked matmul, a
cumulative sum, a projector, a scalar product formula, a dense affine-map
fold, a finite difference, reverse-mode autodiff of an independent program).
"""
import numpy as np
import pytest
import torch

from oracle import wkv7 as o7
from tests.inputs import wkv7_inputs


def _small(B=2, T=12, H=2, N=8, seed=0, **kw):
    kw.setdefault("p_reset", 0.2)
    return wkv7_inputs(B, T, H, N, seed=seed, **kw)


def test_no_ab_is_decayed_linear_attention():
    x = _small(resets=False, lengths=False)
    z = np.zeros_like(x["a"])
    s0 = np.zeros_like(x["s"])
    out_s, y = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], z, z, s0)
    B, T, H, N = x["r"].shape
    logd = -np.exp(x["w"])
    Lc = np.cumsum(logd, axis=1)
    y_ref = np.zeros_like(y)
    for t in range(T):
        for s in range(t + 1):
            kd = x["k"][:, s] * np.exp(Lc[:, t] - Lc[:, s])
            y_ref[:, t] += x["v"][:, s] * np.sum(kd * x["r"][:, t], axis=-1, keepdims=True)
    np.testing.assert_allclose(y, y_ref, rtol=1e-12, atol=1e-12)


def test_no_ab_unit_decay_is_cumsum_of_outer_products():
    x = _small(resets=False, lengths=False)
    z = np.zeros_like(x["a"])
    w = np.full_like(x["w"], -np.inf)       # exp(-exp(-inf)) = 1
    out_s, y = o7.wkv7_base(x["r"], w, x["k"], x["v"], z, z, x["s"])
    outer = np.einsum('bthi,bthj->bthij', x["v"], x["k"])
    S = x["s"][:, None] + np.cumsum(outer, axis=1)
    np.testing.assert_allclose(out_s, S[:, -1], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(y, np.einsum('bthij,bthj->bthi', S, x["r"]), rtol=1e-12, atol=1e-12)


def test_projector_case():
    # v=0, d=1, a=-kappa, b=kappa, |kappa|=1  =>  S_t = S_{t-1}(I - kappa kappa^T): S_t kappa_t = 0, idempotent
    x = _small(resets=False, lengths=False)
    kap = -x["a"]
    kap = kap / np.linalg.norm(kap, axis=-1, keepdims=True)
    w = np.full_like(x["w"], -np.inf)
    zero = np.zeros_like(kap)
    for T in (1, 2, 5):
        sl = lambda q: q[:, :T]
        out_s, y = o7.wkv7_base(sl(kap), sl(w), sl(zero), sl(zero), -sl(kap), sl(kap), x["s"])
        # y_t = S_t r_t with r_t = kappa_t must vanish
        np.testing.assert_allclose(y, 0.0, atol=1e-13)
        P = np.eye(kap.shape[-1])[None, None] - np.einsum('bhi,bhj->bhij', kap[:, T - 1], kap[:, T - 1])
        np.testing.assert_allclose(out_s @ P, out_s, atol=1e-13)


def test_scalar_head_closed_form():
    g = np.random.default_rng(3)
    T = 9
    r, w, k, v, a, b = (g.standard_normal((1, T, 1, 1)) for _ in range(6))
    s0 = g.standard_normal((1, 1, 1, 1))
    out_s, y = o7.wkv7_base(r, w, k, v, a, b, s0)
    m = (np.exp(-np.exp(w)) + a * b).ravel()
    s = s0.item()
    for t in range(T):
        s = s * m[t] + (v * k).ravel()[t]
        assert abs(y.ravel()[t] - s * r.ravel()[t]) < 1e-12
    # product closed form for the final state
    closed = s0.item() * np.prod(m) + sum((v * k).ravel()[i] * np.prod(m[i + 1:]) for i in range(T))
    assert abs(out_s.item() - closed) < 1e-12


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_base_compat_equals_assoc_literal(seed):
    x = _small(seed=seed, T=16, p_reset=0.25, min_len_frac=0.1)
    x["new_starts"][0, 0] = True
    x["length"][0] = 7
    x["new_starts"][0, 7] = True            # Q2 case
    args = (x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"])
    s1, y1 = o7.wkv7_base(*args, compat=True)
    s2, y2 = o7.wkv7_assoc_literal(*args)
    np.testing.assert_allclose(y1, y2, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(s1, s2, rtol=1e-11, atol=1e-12)
    # the two conventions differ exactly where documented
    s3, y3 = o7.wkv7_base(*args, compat=False)
    nxt = np.zeros_like(x["new_starts"])
    nxt[:, :-1] = x["new_starts"][:, 1:]
    np.testing.assert_allclose(y3[~nxt], y2[~nxt], rtol=1e-11, atol=1e-12)
    assert np.all(y2[nxt] == 0) and np.any(y3[nxt] != 0)
    assert np.all(s2[0] == 0) and np.any(s3[0] != 0)


def test_length_zero_conventions():
    x = _small(seed=4, T=6)
    x["length"][:] = 0
    x["new_starts"][:, 0] = [True, False]
    args = (x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"])
    s1, _ = o7.wkv7_base(*args, compat=True)
    s2, _ = o7.wkv7_assoc_literal(*args)
    np.testing.assert_allclose(s1, s2, atol=0)
    s3, _ = o7.wkv7_base(*args, compat=False)
    np.testing.assert_allclose(s3, x["s"], atol=0)          # rwkv7.py:203: out_s starts as s


def test_log_depth_scan_equals_fold():
    x = _small(seed=5, T=13, p_reset=0.2, min_len_frac=0.1)
    args = (x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"])
    s1, y1 = o7.wkv7_assoc_literal(*args)
    s2, y2 = o7.wkv7_assoc_scan(*args, dtype=np.float64)
    np.testing.assert_allclose(y1, y2, rtol=1e-10, atol=1e-11)
    np.testing.assert_allclose(s1, s2, rtol=1e-10, atol=1e-11)


def test_split_sequence_carry_and_length_truncation():
    x = _small(seed=6, T=20, resets=False, lengths=False)
    names = ("r", "w", "k", "v", "a", "b")
    full_s, full_y = o7.wkv7_base(*[x[n] for n in names], x["s"])
    cut = 11
    s_a, y_a = o7.wkv7_base(*[x[n][:, :cut] for n in names], x["s"])
    s_b, y_b = o7.wkv7_base(*[x[n][:, cut:] for n in names], s_a)
    np.testing.assert_allclose(np.concatenate([y_a, y_b], 1), full_y, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(s_b, full_s, rtol=1e-12, atol=1e-12)
    s_len, y_len = o7.wkv7_base(*[x[n] for n in names], x["s"], length=np.array([cut, cut]))
    np.testing.assert_allclose(s_len, s_a, rtol=0, atol=0)
    np.testing.assert_allclose(y_len, full_y, rtol=0, atol=0)      # y is produced for all T


def test_reset_equals_two_independent_runs():
    x = _small(seed=7, T=15, resets=False, lengths=False)
    names = ("r", "w", "k", "v", "a", "b")
    cut = 6
    ns = np.zeros((2, 15), bool)
    ns[:, cut] = True
    s_r, y_r = o7.wkv7_base(*[x[n] for n in names], x["s"], None, ns)
    _, y_a = o7.wkv7_base(*[x[n][:, :cut] for n in names], x["s"])
    s_b, y_b = o7.wkv7_base(*[x[n][:, cut:] for n in names], np.zeros_like(x["s"]))
    np.testing.assert_allclose(y_r, np.concatenate([y_a, y_b], 1), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(s_r, s_b, rtol=1e-12, atol=1e-12)


def test_batch_rows_independent_and_value_row_equivariance():
    x = _small(seed=8)
    names = ("r", "w", "k", "v", "a", "b")
    args = [x[n] for n in names]
    s_all, y_all = o7.wkv7_base(*args, x["s"], x["length"], x["new_starts"])
    s_1, y_1 = o7.wkv7_base(*[q[1:] for q in args], x["s"][1:], x["length"][1:], x["new_starts"][1:])
    np.testing.assert_allclose(y_all[1:], y_1, atol=0)
    np.testing.assert_allclose(s_all[1:], s_1, atol=0)
    perm = np.random.default_rng(0).permutation(x["v"].shape[-1])
    xv = x["v"][..., perm]
    s_p, y_p = o7.wkv7_base(x["r"], x["w"], x["k"], xv, x["a"], x["b"], x["s"][:, :, perm, :], x["length"], x["new_starts"])
    np.testing.assert_allclose(y_p, y_all[..., perm], rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(s_p, s_all[:, :, perm, :], rtol=1e-12, atol=1e-12)


def _loss(x, dy, ds, compat, **over):
    q = dict(x)
    q.update(over)
    out_s, y = o7.wkv7_base(q["r"], q["w"], q["k"], q["v"], q["a"], q["b"], q["s"], q["length"], q["new_starts"], compat=compat)
    return np.sum(y * dy) + np.sum(out_s * ds)


@pytest.mark.parametrize("compat", [False, True])
@pytest.mark.parametrize("case", ["plain", "len_at_reset", "len0"])
def test_bwd_matches_finite_differences(compat, case):
    x = wkv7_inputs(2, 7, 2, 4, seed=11, p_reset=0.3, min_len_frac=0.3)
    x["new_starts"][0, 3] = True
    if case == "len_at_reset":
        x["length"][0] = 3
    if case == "len0":
        x["length"][:] = 0
    dy, ds = x["dy"], x["ds"]
    grads = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], dy, ds, compat=compat)
    g = np.random.default_rng(0)
    eps = 1e-6
    for name, an in zip(("r", "w", "k", "v", "a", "b", "s"), grads):
        for _ in range(12):
            idx = tuple(g.integers(0, n) for n in x[name].shape)
            xp, xm = x[name].copy(), x[name].copy()
            xp[idx] += eps
            xm[idx] -= eps
            fd = (_loss(x, dy, ds, compat, **{name: xp}) - _loss(x, dy, ds, compat, **{name: xm})) / (2 * eps)
            assert abs(fd - an[idx]) < 1e-6 * max(1.0, abs(fd)), (name, idx, fd, an[idx])


def _torch_wkv7(r, w, k, v, a, b, s, length, new_starts):
    """Independent program: dense transition matrices M_t = diag(d_t) + a_t b_t^T, S <- S M_t + v k^T."""
    B, T, H, N = r.shape
    d = torch.exp(-torch.exp(w))
    ys, S, out_s = [], s, s
    for t in range(T):
        keep = (~new_starts[:, t]).to(S.dtype)[:, None, None, None]
        S = S * keep
        M = torch.diag_embed(d[:, t]) + a[:, t, :, :, None] * b[:, t, :, None, :]
        S = S @ M + v[:, t, :, :, None] * k[:, t, :, None, :]
        ys.append((S @ r[:, t, :, :, None]).squeeze(-1))
        snap = (t < length).to(S.dtype)[:, None, None, None]
        out_s = snap * S + (1 - snap) * out_s
    return out_s, torch.stack(ys, 1)


def test_bwd_matches_torch_autograd():
    x = wkv7_inputs(2, 10, 2, 8, seed=12, p_reset=0.2, min_len_frac=0.3)
    tt = {n: torch.tensor(x[n], dtype=torch.float64, requires_grad=True) for n in ("r", "w", "k", "v", "a", "b", "s")}
    out_s, y = _torch_wkv7(tt["r"], tt["w"], tt["k"], tt["v"], tt["a"], tt["b"], tt["s"],
                           torch.tensor(x["length"]), torch.tensor(x["new_starts"]))
    os_np, y_np = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"])
    np.testing.assert_allclose(y.detach().numpy(), y_np, rtol=1e-11, atol=1e-12)
    np.testing.assert_allclose(out_s.detach().numpy(), os_np, rtol=1e-11, atol=1e-12)
    loss = (y * torch.tensor(x["dy"])).sum() + (out_s * torch.tensor(x["ds"])).sum()
    loss.backward()
    grads = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"])
    for name, an in zip(("r", "w", "k", "v", "a", "b", "s"), grads):
        np.testing.assert_allclose(tt[name].grad.numpy(), an, rtol=1e-9, atol=1e-10, err_msg=name)
