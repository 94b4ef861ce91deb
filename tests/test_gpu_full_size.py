"""Size-independent properties at the full benchmark shapes (too large for the float64 oracle): the chunked MFMA
kernels against the sequential fp32 kernels on the same inputs, a split call with the carried state against a
single call, and a reset against a fresh run.  Comparisons stay on the GPU (torch) to keep the host out of it."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def rel_rms(a, b):
    a, b = a.float(), b.float()
    return float((a - b).pow(2).mean().sqrt() / b.pow(2).mean().sqrt().clamp_min(1e-30))


def wkv7_full(B=8, T=4096, H=32, N=64, seed=0, p_reset=1.0 / 1024):
    g = torch.Generator("cuda").manual_seed(seed)
    n = lambda *s: torch.randn(s, device="cuda", generator=g)
    r, k, v, dy = (n(B, T, H, N).bfloat16() for _ in range(4))
    w = (-0.5 + 0.5 * n(B, T, H, N)).bfloat16()
    kap = torch.nn.functional.normalize(n(B, T, H, N), dim=-1)
    a, b = (-kap).bfloat16(), (kap * torch.sigmoid(n(B, T, H, N))).bfloat16()
    s = 0.1 * n(B, H, N, N)
    ns = torch.rand((B, T), device="cuda", generator=g) < p_reset
    length = torch.randint(T // 2, T + 1, (B,), device="cuda", generator=g, dtype=torch.int32)
    return dict(r=r, w=w, k=k, v=v, a=a, b=b, s=s, ns=ns, length=length, dy=dy)


def test_wkv7_forward_and_backward_chunked_equals_sequential_at_the_headline_shape():
    from jaxrwkv_amd import ops
    x = wkv7_full()
    args = (x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["ns"])
    ds = torch.randn_like(x["s"])
    out = {}
    for fs in (False, True):
        new_s, y, sa = ops.wkv7_fwd(*args, compat=True, want_sa=True, force_seq=fs)
        g = ops.wkv7_bwd(*args, x["dy"], sa, ds, compat=True, force_seq=fs)
        out[fs] = (new_s, y, sa) + tuple(g)
    torch.cuda.synchronize()
    names = ("new_s", "y", "sa", "gr", "gw", "gk", "gv", "ga", "gb", "gs")
    # bf16 outputs differ by their rounding (rel-rms 2^-9 ~ 2e-3 each side); the fp32 ones by the operand precision of
    # the chunked kernels: fp16 in the forward pass (state 1-2e-4, sa 3e-4), bf16 hi+lo pairs in the backward sweeps;
    # gb = G^T sa sees the forward's sa through a sum with cancellation (5e-3 on top of its rounding)
    tol = dict(new_s=5e-4, y=4e-3, sa=1e-3, gr=4e-3, gw=6e-3, gk=4e-3, gv=4e-3, ga=4e-3, gb=1e-2, gs=1e-4)
    for n_, c, q in zip(names, out[False], out[True]):
        assert torch.isfinite(c.float()).all(), n_
        assert rel_rms(c, q) < tol[n_], (n_, rel_rms(c, q))


def test_wkv7_fp32_forward_and_backward_chunked_equals_sequential_at_the_headline_shape():
    """fp32 I/O at B=8 T=4096 H=32: the chunked kernels on fp32 matrix instructions against the sequential fp32 kernels,
    forward and all seven cotangents.  Both compute in fp32 throughout, so they agree to a few 1e-6 in relative rms
    (1e-4 for the decay gradient, a running sum over up to 4096 tokens of terms that cancel)."""
    from jaxrwkv_amd import ops
    x = wkv7_full(seed=6)
    args = tuple(x[n].float() for n in "rwkvab") + (x["s"], x["length"], x["ns"])
    dy, ds = x["dy"].float(), torch.randn_like(x["s"])
    out = {}
    for fs in (False, True):
        new_s, y, sa = ops.wkv7_fwd(*args, compat=True, want_sa=True, force_seq=fs)
        g = ops.wkv7_bwd(*args, dy, sa, ds, compat=True, force_seq=fs)
        out[fs] = (new_s, y, sa) + tuple(g)
    torch.cuda.synchronize()
    names = ("new_s", "y", "sa", "gr", "gw", "gk", "gv", "ga", "gb", "gs")
    for n_, c, q in zip(names, out[False], out[True]):
        assert c.dtype == torch.float32 and torch.isfinite(c).all(), n_
        assert rel_rms(c, q) < (1e-4 if n_ == "gw" else 1e-5), (n_, rel_rms(c, q))
    # the cotangents vanish exactly where the forward is cut: dsa-driven ga at every reset token
    assert torch.count_nonzero(out[False][7][x["ns"]]) == 0


def test_wkv7_split_call_with_carried_state_equals_single_call_at_the_headline_shape():
    from jaxrwkv_amd import ops
    x = wkv7_full(seed=1)
    full_s, full_y, _ = ops.wkv7_fwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], None, x["ns"], compat=False)
    h = 2048                                           # a multiple of the chunk length: identical chunking
    sl = lambda t, a, b: t[:, a:b].contiguous()
    s1, y1, _ = ops.wkv7_fwd(*(sl(x[n], 0, h) for n in "rwkvab"), x["s"], None, sl(x["ns"], 0, h), compat=False)
    s2, y2, _ = ops.wkv7_fwd(*(sl(x[n], h, 4096) for n in "rwkvab"), s1, None, sl(x["ns"], h, 4096), compat=False)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([y1, y2], 1), full_y)
    assert torch.equal(s2, full_s)


def test_wkv7_reset_equals_fresh_run_at_the_headline_shape():
    from jaxrwkv_amd import ops
    x = wkv7_full(seed=2)
    ns = torch.zeros_like(x["ns"])
    ns[:, 2048] = True
    _, y, _ = ops.wkv7_fwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], None, ns, compat=False)
    sl = lambda t: t[:, 2048:].contiguous()
    _, y2, _ = ops.wkv7_fwd(*(sl(x[n]) for n in "rwkvab"), torch.zeros_like(x["s"]), None, None, compat=False)
    torch.cuda.synchronize()
    assert torch.equal(y[:, 2048:], y2)


def test_wkv6_chunked_equals_sequential_at_the_benchmark_shape():
    from jaxrwkv_amd import ops
    B, T, H, N = 16, 2048, 32, 64
    g = torch.Generator("cuda").manual_seed(3)
    n = lambda *s: torch.randn(s, device="cuda", generator=g)
    r, k, v, dy = (n(B, T, H, N).bfloat16() for _ in range(4))
    w = (-torch.exp(-0.5 + 0.5 * n(B, T, H, N))).bfloat16()
    u = (0.5 * n(H, N)).bfloat16()
    s = torch.zeros((B, H, N, N), device="cuda")
    ns = torch.rand((B, T), device="cuda", generator=g) < 1.0 / 512
    ds = n(B, H, N, N)
    out = {}
    for fs in (False, True):
        new_s, y = ops.wkv6_fwd(r, k, v, w, u, s, None, ns, compat=True, force_seq=fs)
        out[fs] = (new_s, y) + tuple(ops.wkv6_bwd(r, k, v, w, u, s, None, ns, dy, ds, compat=True, force_seq=fs))
    torch.cuda.synchronize()
    names = ("new_s", "y", "gr", "gk", "gv", "gw", "gu", "gs")
    # the forward's fp16 operands put the state 1-2e-4 (relative rms) from the sequential kernel's
    tol = dict(new_s=5e-4, y=4e-3, gr=4e-3, gk=4e-3, gv=4e-3, gw=6e-3, gu=4e-3, gs=1e-4)
    for n_, c, q in zip(names, out[False], out[True]):
        assert torch.isfinite(c.float()).all(), n_
        assert rel_rms(c, q) < tol[n_], (n_, rel_rms(c, q))


def test_wkv6_fp32_chunked_equals_sequential_at_the_benchmark_shape():
    """fp32 I/O at B=16 T=2048 H=32: the chunked kernels on fp32 matrix instructions against the sequential fp32
    kernels, forward and all six cotangents; both compute in fp32 throughout."""
    from jaxrwkv_amd import ops
    B, T, H, N = 16, 2048, 32, 64
    g = torch.Generator("cuda").manual_seed(7)
    n = lambda *s: torch.randn(s, device="cuda", generator=g)
    r, k, v, dy = (n(B, T, H, N) for _ in range(4))
    w = -torch.exp(-0.5 + 0.5 * n(B, T, H, N))
    u = 0.5 * n(H, N)
    s = 0.1 * n(B, H, N, N)
    ns = torch.rand((B, T), device="cuda", generator=g) < 1.0 / 512
    length = torch.randint(T // 2, T + 1, (B,), device="cuda", generator=g, dtype=torch.int32)
    ds = n(B, H, N, N)
    out = {}
    for fs in (False, True):
        new_s, y = ops.wkv6_fwd(r, k, v, w, u, s, length, ns, compat=True, force_seq=fs)
        out[fs] = (new_s, y) + tuple(ops.wkv6_bwd(r, k, v, w, u, s, length, ns, dy, ds, compat=True, force_seq=fs))
    torch.cuda.synchronize()
    names = ("new_s", "y", "gr", "gk", "gv", "gw", "gu", "gs")
    for n_, c, q in zip(names, out[False], out[True]):
        assert c.dtype == torch.float32 and torch.isfinite(c).all(), n_
        assert rel_rms(c, q) < (1e-4 if n_ == "gw" else 1e-5), (n_, rel_rms(c, q))


def test_wkv4_split_call_equals_single_call_at_the_benchmark_shape():
    from jaxrwkv_amd import ops
    B, T, C = 32, 4096, 2560
    g = torch.Generator("cuda").manual_seed(4)
    k = torch.randn((B, T, C), device="cuda", generator=g)
    v = torch.randn((B, T, C), device="cuda", generator=g)
    w = -torch.exp(torch.randn(C, device="cuda", generator=g))
    u = 0.5 * torch.randn(C, device="cuda", generator=g)
    s = torch.zeros((B, 3, C), device="cuda")
    s[:, 2] = -1e38
    full_s, full_y = ops.wkv4_fwd(w, u, k, v, s, None, None, compat=False)
    s1, y1 = ops.wkv4_fwd(w, u, k[:, :1000].contiguous(), v[:, :1000].contiguous(), s, None, None, compat=False)
    s2, y2 = ops.wkv4_fwd(w, u, k[:, 1000:].contiguous(), v[:, 1000:].contiguous(), s1, None, None, compat=False)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([y1, y2], 1), full_y)
    assert torch.equal(s2, full_s)


def test_wkv7_prefill_shape_of_the_1p5b_config():
    """BASELINE configs[4], prefill: the op at B=16, T=4096, H=32, bf16, new_starts ~ Bernoulli(1/2048).  Chunked
    against sequential kernel, and a split call with the carried state against the single call."""
    from jaxrwkv_amd import ops
    x = wkv7_full(B=16, seed=5, p_reset=1.0 / 2048)
    args = [x[n] for n in "rwkvab"]
    new_s, y, _ = ops.wkv7_fwd(*args, x["s"], x["length"], x["ns"], compat=True)
    seq_s, seq_y, _ = ops.wkv7_fwd(*args, x["s"], x["length"], x["ns"], compat=True, force_seq=True)
    torch.cuda.synchronize()
    assert torch.isfinite(y.float()).all() and torch.isfinite(new_s).all()
    assert rel_rms(y, seq_y) < 4e-3, rel_rms(y, seq_y)
    assert rel_rms(new_s, seq_s) < 2e-3, rel_rms(new_s, seq_s)
    # y is exactly zero where the associative form defines it so, in both kernels
    nxt = torch.zeros_like(x["ns"])
    nxt[:, :-1] = x["ns"][:, 1:]
    assert torch.count_nonzero(y[nxt]) == 0 and torch.count_nonzero(seq_y[nxt]) == 0
    del seq_s, seq_y
    full_s, full_y, _ = ops.wkv7_fwd(*args, x["s"], None, x["ns"], compat=False)
    h = 2048
    sl = lambda t, a, b: t[:, a:b].contiguous()
    s1, y1, _ = ops.wkv7_fwd(*(sl(t, 0, h) for t in args), x["s"], None, sl(x["ns"], 0, h), compat=False)
    s2, y2, _ = ops.wkv7_fwd(*(sl(t, h, 4096) for t in args), s1, None, sl(x["ns"], h, 4096), compat=False)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([y1, y2], 1), full_y)
    assert torch.equal(s2, full_s)


@pytest.mark.parametrize("st", [torch.float32, torch.bfloat16])
def test_wkv7_decode_shape_of_the_1p5b_config(st):
    """BASELINE configs[4], decode: one token for B=256 sequences x 32 heads from a carried state, against the float64
    oracle (bf16 inputs; fp32 state to the fp32 bar, bf16 state and y within one bf16 ulp)."""
    import numpy as np
    from jaxrwkv_amd import ops
    from oracle import wkv7 as o7
    from tests.gpu_util import assert_close, dev, host
    from tests.inputs import bf16_round, wkv7_inputs
    x = wkv7_inputs(256, 1, 32, 64, seed=9, bf16=True, resets=False, lengths=False, s_scale=1.0)
    x["new_starts"][::7, 0] = True                                  # some sequences start afresh at this token
    if st == torch.bfloat16:
        x["s"] = bf16_round(x["s"]).astype(np.float64)
    ref_s, ref_y = o7.wkv7_base(*[x[n] for n in "rwkvab"], x["s"], x["length"], x["new_starts"], compat=True)
    t = {n: dev(x[n], torch.bfloat16) for n in "rwkvab"}
    new_s, y, _ = ops.wkv7_fwd(*[t[n] for n in "rwkvab"], dev(x["s"], st), dev(x["length"]), dev(x["new_starts"]), compat=True)
    torch.cuda.synchronize()
    assert_close("y", host(y), ref_y, rtol=2.0 ** -8, atol=1e-5)
    if st == torch.float32:
        assert_close("new_s", host(new_s), ref_s)
    else:
        assert_close("new_s", host(new_s), ref_s, rtol=2.0 ** -8, atol=1e-6)


def test_wkv7_fp32_chunked_equals_sequential_and_split_call_at_the_headline_shape():
    """fp32 I/O at B=8 T=4096 H=32: the chunked kernel on fp32 matrix instructions against the sequential fp32 kernel
    at the fp32 bar (rtol 1e-4, atol 1e-5 of the tensor's rms scale), and a split call with the carried state against
    the single call, bit for bit."""
    from jaxrwkv_amd import ops
    x = wkv7_full(seed=5)
    f = {n: x[n].float() for n in "rwkvab"}
    args = tuple(f[n] for n in "rwkvab") + (x["s"], x["length"], x["ns"])
    a = ops.wkv7_fwd(*args, compat=True, want_sa=True)
    b = ops.wkv7_fwd(*args, compat=True, want_sa=True, force_seq=True)
    torch.cuda.synchronize()
    for name, c, q in zip(("new_s", "y", "sa"), a, b):
        assert c.dtype == torch.float32 and torch.isfinite(c).all(), name
        scale = float(q.pow(2).mean().sqrt())
        excess = ((c - q).abs() - 1e-4 * q.abs()).max()
        assert float(excess) < 1e-5 * max(1.0, scale), (name, float(excess), scale)
    h = 2048
    sl = lambda t, lo, hi: t[:, lo:hi].contiguous()
    full_s, full_y, _ = ops.wkv7_fwd(*(f[n] for n in "rwkvab"), x["s"], None, x["ns"], compat=False)
    s1, y1, _ = ops.wkv7_fwd(*(sl(f[n], 0, h) for n in "rwkvab"), x["s"], None, sl(x["ns"], 0, h), compat=False)
    s2, y2, _ = ops.wkv7_fwd(*(sl(f[n], h, 4096) for n in "rwkvab"), s1, None, sl(x["ns"], h, 4096), compat=False)
    torch.cuda.synchronize()
    assert torch.equal(torch.cat([y1, y2], 1), full_y) and torch.equal(s2, full_s)


def test_wkv4_backward_with_forward_checkpoints_at_the_benchmark_shape():
    """B=32 T=4096 C=2560 fp32: the forward that keeps the checkpoints returns the plain forward's bits, and the
    backward that takes them returns the bits of the backward with its own checkpoint pass."""
    from jaxrwkv_amd import ops
    B, T, C = 32, 4096, 2560
    g = torch.Generator("cuda").manual_seed(6)
    k = torch.randn((B, T, C), device="cuda", generator=g)
    v = torch.randn((B, T, C), device="cuda", generator=g)
    gy = torch.randn((B, T, C), device="cuda", generator=g)
    w = -torch.exp(torch.randn(C, device="cuda", generator=g))
    u = 0.5 * torch.randn(C, device="cuda", generator=g)
    s = torch.zeros((B, 3, C), device="cuda")
    s[:, 2] = -1e38
    length = torch.randint(1024, T + 1, (B,), device="cuda", generator=g, dtype=torch.int32)
    ns = torch.rand((B, T), device="cuda", generator=g) < 1.0 / 1024
    plain = ops.wkv4_fwd(w, u, k, v, s, length, ns)
    new_s, y, ck = ops.wkv4_fwd(w, u, k, v, s, length, ns, want_ckpt=True)
    assert torch.equal(new_s, plain[0]) and torch.equal(y, plain[1])
    own = ops.wkv4_bwd(w, u, k, v, s, length, ns, gy)
    taken = ops.wkv4_bwd(w, u, k, v, s, length, ns, gy, ckpt=ck)
    torch.cuda.synchronize()
    for p_, q_ in zip(own, taken):
        assert torch.isfinite(p_.float()).all() and torch.equal(p_, q_)
