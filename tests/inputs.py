"""Seeded synthetic inputs for the WKV ops, in the distributions the benchmark configs name."""
import numpy as np


def bf16_round(x):
    """Round float arrays to the nearest bfloat16 (ties to even), returned as float32."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    u = x.view(np.uint32).astype(np.uint64)
    u = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    return u.astype(np.uint32).view(np.float32)


def wkv7_inputs(B, T, H, N=64, seed=0, p_reset=1.0 / 1024, min_len_frac=0.5, s_scale=0.1, bf16=False,
                resets=True, lengths=True):
    """r,k,v ~ N(0,1); w = x ~ N(-0.5, 0.5) (the op applies exp(-exp(x))); kappa = unit N(0,1) per head;
    a = -kappa; b = kappa * sigmoid(N(0,1)); s ~ N(0, s_scale); new_starts ~ Bernoulli(p); length ~ U{T*frac..T}."""
    g = np.random.default_rng(seed)
    r = g.standard_normal((B, T, H, N))
    k = g.standard_normal((B, T, H, N))
    v = g.standard_normal((B, T, H, N))
    w = -0.5 + 0.5 * g.standard_normal((B, T, H, N))
    kap = g.standard_normal((B, T, H, N))
    kap /= np.linalg.norm(kap, axis=-1, keepdims=True)
    a = -kap
    b = kap / (1.0 + np.exp(-g.standard_normal((B, T, H, N))))
    s = s_scale * g.standard_normal((B, H, N, N))
    ns = (g.random((B, T)) < p_reset) if resets else np.zeros((B, T), bool)
    lo = max(1, int(T * min_len_frac))
    length = g.integers(lo, T + 1, size=(B,)) if lengths else np.full((B,), T)
    dy = g.standard_normal((B, T, H, N))
    ds = g.standard_normal((B, H, N, N))
    arrs = dict(r=r, w=w, k=k, v=v, a=a, b=b, dy=dy)
    if bf16:
        arrs = {n: bf16_round(x).astype(np.float64) for n, x in arrs.items()}
    arrs.update(s=s.astype(np.float32).astype(np.float64), ds=ds.astype(np.float32).astype(np.float64),
                new_starts=ns, length=length.astype(np.int32))
    if not bf16:
        for n in ("r", "w", "k", "v", "a", "b", "dy"):
            arrs[n] = arrs[n].astype(np.float32).astype(np.float64)
    return arrs


def wkv6_inputs(B, T, H, N=64, seed=0, p_reset=1.0 / 512, bf16=False, zero_state=False, resets=True, lengths=True):
    """r,k,v ~ N(0,1); log-decay w = -exp(N(-0.5,0.5)); u ~ N(0,0.5) per head-channel."""
    g = np.random.default_rng(seed)
    r = g.standard_normal((B, T, H, N))
    k = g.standard_normal((B, T, H, N))
    v = g.standard_normal((B, T, H, N))
    w = -np.exp(-0.5 + 0.5 * g.standard_normal((B, T, H, N)))
    u = 0.5 * g.standard_normal((H, N))
    s = np.zeros((B, H, N, N)) if zero_state else 0.1 * g.standard_normal((B, H, N, N))
    ns = (g.random((B, T)) < p_reset) if resets else np.zeros((B, T), bool)
    length = g.integers(max(1, T // 2), T + 1, size=(B,)) if lengths else np.full((B,), T)
    dy = g.standard_normal((B, T, H, N))
    ds = g.standard_normal((B, H, N, N))
    arrs = dict(r=r, k=k, v=v, w=w, u=u, dy=dy)
    rnd = bf16_round if bf16 else (lambda x: x.astype(np.float32))
    arrs = {n: rnd(x).astype(np.float64) for n, x in arrs.items()}
    arrs.update(s=s.astype(np.float32).astype(np.float64), ds=ds.astype(np.float32).astype(np.float64),
                new_starts=ns, length=length.astype(np.int32))
    return arrs


def wkv4_inputs(B, T, C, seed=0, p_reset=0.0, min_len=None, default_state=True):
    """k,v ~ N(0,1); w = -exp(N(0,1)); u ~ N(0,0.5); state (0,0,-1e38) or random."""
    g = np.random.default_rng(seed)
    k = g.standard_normal((B, T, C))
    v = g.standard_normal((B, T, C))
    w = -np.exp(g.standard_normal((C,)))
    u = 0.5 * g.standard_normal((C,))
    if default_state:
        s = np.zeros((B, 3, C))
        s[:, 2] = -1e38
    else:
        s = np.stack([g.standard_normal((B, C)), np.abs(g.standard_normal((B, C))) + 0.5,
                      g.standard_normal((B, C))], axis=1)
    ns = g.random((B, T)) < p_reset
    lo = max(1, T // 4) if min_len is None else min_len
    length = g.integers(lo, T + 1, size=(B,))
    f = lambda x: x.astype(np.float32).astype(np.float64)
    return dict(k=f(k), v=f(v), w=f(w), u=f(u), s=f(s), new_starts=ns, length=length.astype(np.int32))
