"""The chunked kernels' bounded hand-shake fails loudly: with HIPRWKV_DEBUG_DROP_PUBLISH the producer of the last
chunk never publishes it, the consumers' wait runs out, every wave still ends normally (the launch returns, later
launches work), all outputs of every (sequence, head) are NaN and the failure counter advances by B*H per kernel."""
import os

import pytest
import torch

# the library accepts the test hook only in a process that asks for it (read at the first call that carries the flag)
os.environ["HIPRWKV_ENABLE_DEBUG_FLAGS"] = "1"

pytestmark = pytest.mark.gpu

B, T, H, N = 2, 80, 3, 64


def inputs7(seed=0):
    g = torch.Generator("cuda").manual_seed(seed)
    n = lambda *s: torch.randn(s, device="cuda", generator=g)
    r, k, v, dy = (n(B, T, H, N).bfloat16() for _ in range(4))
    w = (-0.5 + 0.5 * n(B, T, H, N)).bfloat16()
    kap = torch.nn.functional.normalize(n(B, T, H, N), dim=-1)
    a, b = (-kap).bfloat16(), (kap * torch.sigmoid(n(B, T, H, N))).bfloat16()
    return (r, w, k, v, a, b, 0.1 * n(B, H, N, N), None, None), dy, n(B, H, N, N)


def all_nan(t):
    return bool(torch.isnan(t.float()).all())


def test_wkv7_forward_and_backward_poison_their_outputs_and_count():
    from jaxrwkv_amd import _lib, ops
    args, dy, ds = inputs7()
    good = ops.wkv7_fwd(*args, want_sa=True)
    before = ops.handshake_failures()
    new_s, y, sa = ops.wkv7_fwd(*args, want_sa=True, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == B * H
    assert all_nan(new_s) and all_nan(y) and all_nan(sa)
    before = ops.handshake_failures()
    grads = ops.wkv7_bwd(*args, dy, good[2], ds, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == 3 * B * H          # three sweeps
    for g in grads:
        assert all_nan(g)
    # the kernels ended normally: the same launches without the hook work and report nothing
    before = ops.handshake_failures()
    again = ops.wkv7_fwd(*args, want_sa=True)
    g2 = ops.wkv7_bwd(*args, dy, again[2], ds)
    assert ops.handshake_failures() == before
    for a_, b_ in zip(again, good):
        assert torch.equal(a_, b_)
    assert all(bool(torch.isfinite(g.float()).all()) for g in g2)


def test_wkv7_forward_without_the_residual_poisons_its_outputs_and_counts():
    """The launch without `sa` is an instantiation of its own (its consumers store y themselves; with `sa` the
    producers write it out): the same failure path, checked separately."""
    from jaxrwkv_amd import _lib, ops
    args, _, _ = inputs7(seed=1)
    good = ops.wkv7_fwd(*args, want_sa=False)
    before = ops.handshake_failures()
    new_s, y, sa = ops.wkv7_fwd(*args, want_sa=False, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert sa is None
    assert ops.handshake_failures() - before == B * H
    assert all_nan(new_s) and all_nan(y)
    before = ops.handshake_failures()
    again = ops.wkv7_fwd(*args, want_sa=False)
    assert ops.handshake_failures() == before
    assert torch.equal(again[0], good[0]) and torch.equal(again[1], good[1])
    # both instantiations give the same y and state
    with_sa = ops.wkv7_fwd(*args, want_sa=True)
    assert torch.equal(with_sa[0], good[0]) and torch.equal(with_sa[1], good[1])


def test_wkv6_forward_and_backward_poison_their_outputs_and_count():
    from jaxrwkv_amd import _lib, ops
    g = torch.Generator("cuda").manual_seed(1)
    n = lambda *s: torch.randn(s, device="cuda", generator=g)
    r, k, v, dy = (n(B, T, H, N).bfloat16() for _ in range(4))
    w = (-torch.exp(-0.5 + 0.5 * n(B, T, H, N))).bfloat16()
    u = (0.5 * n(H, N)).bfloat16()
    s, ds = 0.1 * n(B, H, N, N), n(B, H, N, N)
    good = ops.wkv6_fwd(r, k, v, w, u, s)
    before = ops.handshake_failures()
    new_s, y = ops.wkv6_fwd(r, k, v, w, u, s, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == B * H
    assert all_nan(new_s) and all_nan(y)
    before = ops.handshake_failures()
    grads = ops.wkv6_bwd(r, k, v, w, u, s, None, None, dy, ds, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == 2 * B * H          # two sweeps
    for t in grads:
        assert all_nan(t)
    before = ops.handshake_failures()
    again = ops.wkv6_fwd(r, k, v, w, u, s)
    assert ops.handshake_failures() == before
    assert torch.equal(again[0], good[0]) and torch.equal(again[1], good[1])


def test_wkv7_fp32_forward_poisons_its_outputs_and_counts():
    from jaxrwkv_amd import _lib, ops
    args, _, _ = inputs7(seed=2)
    args = tuple(t.float() if isinstance(t, torch.Tensor) else t for t in args)
    good = ops.wkv7_fwd(*args, want_sa=True)
    before = ops.handshake_failures()
    new_s, y, sa = ops.wkv7_fwd(*args, want_sa=True, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == B * H
    assert y.dtype == torch.float32 and all_nan(new_s) and all_nan(y) and all_nan(sa)
    before = ops.handshake_failures()
    again = ops.wkv7_fwd(*args, want_sa=True)
    assert ops.handshake_failures() == before
    for a_, b_ in zip(again, good):
        assert torch.equal(a_, b_)


def test_wkv7_fp32_backward_poisons_its_outputs_and_counts():
    from jaxrwkv_amd import _lib, ops
    args, dy, ds = inputs7(seed=3)
    args = tuple(t.float() if isinstance(t, torch.Tensor) else t for t in args)
    dy = dy.float()
    good = ops.wkv7_fwd(*args, want_sa=True)
    ref = ops.wkv7_bwd(*args, dy, good[2], ds)
    before = ops.handshake_failures()
    grads = ops.wkv7_bwd(*args, dy, good[2], ds, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == 3 * B * H          # three sweeps
    for g in grads:
        assert g.dtype == torch.float32 and all_nan(g)
    before = ops.handshake_failures()
    again = ops.wkv7_bwd(*args, dy, good[2], ds)
    assert ops.handshake_failures() == before
    for a_, b_ in zip(again, ref):
        assert torch.equal(a_, b_)


def test_wkv6_fp32_forward_and_backward_poison_their_outputs_and_count():
    from jaxrwkv_amd import _lib, ops
    g = torch.Generator("cuda").manual_seed(4)
    n = lambda *s: torch.randn(s, device="cuda", generator=g)
    r, k, v, dy = (n(B, T, H, N) for _ in range(4))
    w = -torch.exp(-0.5 + 0.5 * n(B, T, H, N))
    u = 0.5 * n(H, N)
    s, ds = 0.1 * n(B, H, N, N), n(B, H, N, N)
    good = ops.wkv6_fwd(r, k, v, w, u, s)
    ref = ops.wkv6_bwd(r, k, v, w, u, s, None, None, dy, ds)
    before = ops.handshake_failures()
    new_s, y = ops.wkv6_fwd(r, k, v, w, u, s, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == B * H
    assert y.dtype == torch.float32 and all_nan(new_s) and all_nan(y)
    before = ops.handshake_failures()
    grads = ops.wkv6_bwd(r, k, v, w, u, s, None, None, dy, ds, debug_flags=_lib.DEBUG_DROP_PUBLISH)
    assert ops.handshake_failures() - before == 2 * B * H          # two sweeps
    for t in grads:
        assert all_nan(t)
    before = ops.handshake_failures()
    again = ops.wkv6_fwd(r, k, v, w, u, s)
    g2 = ops.wkv6_bwd(r, k, v, w, u, s, None, None, dy, ds)
    assert ops.handshake_failures() == before
    assert torch.equal(again[0], good[0]) and torch.equal(again[1], good[1])
    for a_, b_ in zip(g2, ref):
        assert torch.equal(a_, b_)
