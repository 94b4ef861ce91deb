"""RWKV-5 / RWKV-5.2 plug-in (HipRWKV.inner_loop over the WKV6 kernels) against the float64 RWKV-5 oracle."""
import numpy as np
import pytest
import torch

from oracle import wkv5 as o5
from tests.gpu_util import assert_close, dev, host
from tests.inputs import bf16_round

pytestmark = pytest.mark.gpu


def inputs(B, T, H, seed, per_channel, bf16):
    g = np.random.default_rng(seed)
    N = 64
    rnd = (lambda x: bf16_round(x).astype(np.float64)) if bf16 else (lambda x: x.astype(np.float32).astype(np.float64))
    r, k, v = (rnd(g.standard_normal((B, T, H, N))) for _ in range(3))
    # decays down to e^-e = 0.066 per token (RWKV-5 models initialise 0.69 .. 0.9975)
    w = rnd(np.exp(-np.exp(np.clip(g.standard_normal((H, N if per_channel else 1, 1)) - 1.0, None, 1.0))))
    u = rnd(np.exp(0.3 * g.standard_normal((H, N if per_channel else 1, 1))))
    s = (0.1 * g.standard_normal((B, H, N, N))).astype(np.float32).astype(np.float64)
    ns = g.random((B, T)) < 0.03
    length = g.integers(max(1, T // 2), T + 1, size=(B,))
    return r, k, v, w, u, s, length, ns


@pytest.mark.parametrize("per_channel", [False, True])
def test_fp32_batched_and_unbatched(per_channel):
    from jaxrwkv_amd.rwkv5 import HipRWKV
    r, k, v, w, u, s, length, ns = inputs(2, 70, 2, 3, per_channel, False)
    ref_s, ref_y = o5.wkv5_base(r, k, v, w, u, s, length, ns, compat=True)
    new_s, y = HipRWKV.inner_loop(dev(r), dev(k), dev(v), dev(w), dev(u), dev(s), dev(length), dev(ns))
    assert_close("y", host(y), ref_y)
    assert_close("new_s", host(new_s), ref_s)
    new_s, y = HipRWKV.inner_loop(dev(r[0]), dev(k[0]), dev(v[0]), dev(w), dev(u), dev(s[0]), int(length[0]), dev(ns[0]))
    assert_close("y", host(y), ref_y[0])
    assert_close("new_s", host(new_s), ref_s[0])


@pytest.mark.parametrize("per_channel", [False, True])
def test_bf16(per_channel):
    from jaxrwkv_amd.rwkv5 import HipRWKV
    r, k, v, w, u, s, length, ns = inputs(2, 200, 2, 4, per_channel, True)
    ref_s, ref_y = o5.wkv5_base(r, k, v, w, u, s, length, ns, compat=True)
    bf = torch.bfloat16
    new_s, y = HipRWKV.inner_loop(dev(r, bf), dev(k, bf), dev(v, bf), dev(w, bf), dev(u, bf), dev(s), dev(length), dev(ns))
    # log(w) is rounded to bf16 once more: 2^-9 |log w| per step on the decay
    assert_close("y", host(y), ref_y, rtol=2.0 ** -6, atol=2e-2, scale_atol=True)
    assert_close("new_s", host(new_s), bf16_round(ref_s).astype(np.float64), rtol=2.0 ** -6, atol=2e-2, scale_atol=True)


@pytest.mark.parametrize("dtype,T,force_seq", [(torch.bfloat16, 100, False), (torch.float32, 50, False),
                                               (torch.bfloat16, 40, True), (torch.bfloat16, 5, False)])
def test_shared_decay_equals_the_broadcast_one(dtype, T, force_seq):
    """HIPRWKV_W_PER_HEAD: an (H,N) log decay gives bit-identical outputs and cotangents to the same decay
    materialised per token, on the chunked, sequential and small-T kernels; its own cotangent is the per-token one
    summed over batch and tokens."""
    from jaxrwkv_amd import ops
    B, H, N = 2, 3, 64
    g = torch.Generator("cuda").manual_seed(7)
    n = lambda *s: torch.randn(s, device="cuda", generator=g)
    r, k, v, dy = (n(B, T, H, N).to(dtype) for _ in range(4))
    logw = (-torch.exp(n(H, N) - 1.0)).to(dtype)
    u = (0.5 * n(H, N)).to(dtype)
    s, ds = 0.1 * n(B, H, N, N), n(B, H, N, N)
    ns = torch.rand((B, T), device="cuda", generator=g) < 0.05
    length = torch.tensor([T, max(1, T // 2)], device="cuda", dtype=torch.int32)
    wide = logw[None, None].expand(B, T, H, N).contiguous()
    a = ops.wkv6_fwd(r, k, v, logw, u, s, length, ns, force_seq=force_seq)
    b = ops.wkv6_fwd(r, k, v, wide, u, s, length, ns, force_seq=force_seq)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    ga = ops.wkv6_bwd(r, k, v, logw, u, s, length, ns, dy, ds, force_seq=force_seq)
    gb = ops.wkv6_bwd(r, k, v, wide, u, s, length, ns, dy, ds, force_seq=force_seq)
    for i in (0, 1, 2, 4, 5):
        assert torch.equal(ga[i], gb[i]), i
    assert ga[3].shape == (H, N)
    torch.testing.assert_close(ga[3].float(), gb[3].float().sum((0, 1)), rtol=2.0 ** -7 if dtype == torch.bfloat16 else 1e-5,
                               atol=1e-5)


def test_rwkv5_plugin_gradients_reach_the_decay():
    from jaxrwkv_amd.rwkv5 import HipRWKV
    r, k, v, w, u, s, length, ns = inputs(2, 48, 2, 5, True, False)
    t = [dev(x).requires_grad_() for x in (r, k, v, w, u, s)]
    new_s, y = HipRWKV.inner_loop(*t, dev(length), dev(ns))
    (y.sum() + new_s.sum()).backward()
    assert t[3].grad is not None and t[3].grad.shape == t[3].shape and bool(torch.isfinite(t[3].grad).all())
    assert float(t[3].grad.abs().max()) > 0
