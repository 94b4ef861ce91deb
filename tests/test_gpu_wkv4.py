"""WKV4 parity on the GPU: the HIP path (through the C ABI) against the float64 oracle and the committed fixture."""
import os

import numpy as np
import pytest
import torch

from oracle import wkv4 as o4
from tests.gpu_util import assert_close, dev, host
from tests.inputs import wkv4_inputs

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "wkv4_small.npz")


def run_fwd(x, compat, dtype=torch.float32):
    from jaxrwkv_amd import ops
    new_s, y = ops.wkv4_fwd(dev(x["w"], dtype), dev(x["u"], dtype), dev(x["k"], dtype), dev(x["v"], dtype),
                            dev(x["s"], dtype), dev(x["length"]), dev(x["new_starts"]), compat=compat)
    torch.cuda.synchronize()
    return host(new_s), host(y)


def state_close(got, ref):
    """(aa,bb,pp) compared raw, with pp = -1e30/-1e38 ('minus infinity') entries compared as such."""
    assert_close("aa", got[:, 0], ref[:, 0])
    assert_close("bb", got[:, 1], ref[:, 1])
    big = ref[:, 2] < -1e29
    assert np.array_equal(got[:, 2] < -1e29, big)
    assert_close("pp", got[:, 2][~big], ref[:, 2][~big])


@pytest.mark.parametrize("compat", [True, False])
def test_fp32_golden_fixture(compat):
    z = dict(np.load(GOLD))
    new_s, y = run_fwd(z, compat)
    assert_close("y", y, z[f"y_c{int(compat)}"])
    state_close(new_s, z[f"new_s_c{int(compat)}"])


@pytest.mark.parametrize("B,T,C,seed", [(1, 1, 64, 0), (2, 17, 100, 1), (3, 130, 257, 2), (2, 515, 64, 3)])
@pytest.mark.parametrize("compat", [True, False])
@pytest.mark.parametrize("default_state", [True, False])
def test_fp32_forward_shapes(B, T, C, seed, compat, default_state):
    x = wkv4_inputs(B, T, C, seed=seed, p_reset=0.05, default_state=default_state, min_len=1)
    if T > 4:
        x["new_starts"][0, 0] = True
        x["length"][0] = T // 2
        x["new_starts"][0, T // 2] = True
    ref_s, ref_y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=compat)
    new_s, y = run_fwd(x, compat)
    assert_close("y", y, ref_y)
    state_close(new_s, ref_s)


@pytest.mark.parametrize("T,C,p_reset", [(200, 100, 0.0), (333, 64, 0.004), (96, 257, 0.0), (64, 65, 0.01)])
def test_fp32_blocks_without_resets(T, C, p_reset):
    """Long runs of tokens with no reset, sequence end or `length` in them: the kernel's check-free blocks, next
    to blocks that have one; channel counts that leave part of the last wavefront without a channel of its own."""
    x = wkv4_inputs(2, T, C, seed=11 + T, p_reset=p_reset, default_state=False, min_len=T // 2)
    ref_s, ref_y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=True)
    new_s, y = run_fwd(x, True)
    assert_close("y", y, ref_y)
    state_close(new_s, ref_s)


def test_fp32_without_new_starts_pointer():
    from jaxrwkv_amd import ops
    x = wkv4_inputs(2, 150, 70, seed=21, default_state=True, min_len=150)
    ref_s, ref_y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=True)
    f = torch.float32
    new_s, y = ops.wkv4_fwd(dev(x["w"], f), dev(x["u"], f), dev(x["k"], f), dev(x["v"], f), dev(x["s"], f), None, None)
    torch.cuda.synchronize()
    assert_close("y", host(y), ref_y)
    state_close(host(new_s), ref_s)


def test_large_k_is_stable():
    x = wkv4_inputs(2, 64, 64, seed=5)
    x["k"] = x["k"] * 60.0
    ref_s, ref_y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"])
    new_s, y = run_fwd(x, True)
    assert np.all(np.isfinite(y))
    assert_close("y", y, ref_y, rtol=1e-4, atol=1e-4)


def test_plugin_class_applies_decay_and_receptance():
    from jaxrwkv_amd.rwkv4 import HipRWKV
    x = wkv4_inputs(1, 30, 64, seed=6, p_reset=0.05, default_state=False)
    g = np.random.default_rng(0)
    r = g.random((30, 64))
    td = np.log(-x["w"])
    new_s, out = HipRWKV.inner_loop(dev(r), dev(x["k"][0]), dev(x["v"][0]), dev(td), dev(x["u"]), dev(x["s"][0]),
                                    int(x["length"][0]), dev(x["new_starts"][0]))
    ref_s, ref_y = o4.wkv4_assoc_literal(r[None], x["k"], x["v"], td, x["u"], x["s"], x["length"], x["new_starts"])
    assert_close("out", host(out), ref_y[0])
    state_close(host(new_s)[None], ref_s)


def run_bwd(x, gy, gs, compat):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n]).requires_grad_() for n in ("w", "u", "k", "v", "s")}
    new_s, y = ops.wkv4(t["w"], t["u"], t["k"], t["v"], t["s"], dev(x["length"]), dev(x["new_starts"]), compat=compat)
    # the constant "minus infinity" of a reset state is excluded from the loss, as in the oracle's check
    mask = (new_s > -1e29).float()
    ((y * dev(gy)).sum() + (new_s * mask * dev(gs)).sum()).backward()
    torch.cuda.synchronize()
    return [host(t[n].grad) for n in ("w", "u", "k", "v", "s")]


@pytest.mark.parametrize("compat", [True, False])
@pytest.mark.parametrize("B,T,C,seed", [(2, 40, 64, 31), (3, 130, 100, 32), (1, 1, 64, 33)])
def test_fp32_backward(B, T, C, seed, compat):
    x = wkv4_inputs(B, T, C, seed=seed, p_reset=0.04, default_state=False, min_len=1)
    if T > 4:
        x["length"][0] = T // 2
        x["new_starts"][0, T // 2] = True
    g = np.random.default_rng(seed)
    gy, gs = g.standard_normal(x["k"].shape), g.standard_normal(x["s"].shape)
    ref_s, _ = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=compat)
    gs_eff = np.where(ref_s > -1e29, gs, 0.0)
    gw, gu, gk, gv, gsi = o4.wkv4_ffi_bwd(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], gy, gs_eff, compat=compat)
    got = run_bwd(x, gy, gs, compat)
    for name, g_, rf in zip(("w", "u", "k", "v", "s"), got, (gw.sum(0), gu.sum(0), gk, gv, gsi)):
        assert_close("g" + name, g_, rf, rtol=1e-4, atol=2e-5, scale_atol=True)


def test_backward_length_zero_and_default_state():
    x = wkv4_inputs(2, 20, 64, seed=34, p_reset=0.1)
    x["length"][:] = 0
    g = np.random.default_rng(1)
    gy, gs = g.standard_normal(x["k"].shape), g.standard_normal(x["s"].shape)
    for compat in (True, False):
        ref_s, _ = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=compat)
        gs_eff = np.where(ref_s > -1e29, gs, 0.0)
        gw, gu, gk, gv, gsi = o4.wkv4_ffi_bwd(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], gy, gs_eff, compat=compat)
        got = run_bwd(x, gy, gs, compat)
        for name, g_, rf in zip(("w", "u", "k", "v", "s"), got, (gw.sum(0), gu.sum(0), gk, gv, gsi)):
            assert_close("g" + name, g_, rf, rtol=1e-4, atol=2e-5, scale_atol=True)


def bf16_inputs(B, T, C, seed):
    """Inputs and state rounded to bf16, so that the float64 oracle and the kernel start from the same numbers."""
    from tests.inputs import bf16_round
    x = wkv4_inputs(B, T, C, seed=seed, p_reset=0.04, default_state=False, min_len=1)
    for n in ("w", "u", "k", "v", "s"):
        x[n] = bf16_round(x[n]).astype(np.float64)
    if T > 4:
        x["length"][0] = T // 2
        x["new_starts"][0, T // 2] = True
    return x


@pytest.mark.parametrize("compat", [True, False])
@pytest.mark.parametrize("B,T,C,seed", [(2, 40, 64, 41), (3, 130, 100, 42), (2, 515, 257, 43)])
def test_bf16_forward(B, T, C, seed, compat):
    """bf16 I/O (the reference's wkv4-fwd-bf16 target, rwkv4.py:396-397): fp32 arithmetic on bf16 inputs, outputs and
    state rounded once: within one bf16 ulp (2^-8 relative) of the float64 oracle."""
    x = bf16_inputs(B, T, C, seed)
    ref_s, ref_y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=compat)
    new_s, y = run_fwd(x, compat, torch.bfloat16)
    assert_close("y", y, ref_y, rtol=2.0 ** -8, atol=1e-6)
    assert_close("aa", new_s[:, 0], ref_s[:, 0], rtol=2.0 ** -8, atol=1e-6)
    assert_close("bb", new_s[:, 1], ref_s[:, 1], rtol=2.0 ** -8, atol=1e-6)
    big = ref_s[:, 2] < -1e29
    assert np.array_equal(new_s[:, 2] < -1e29, big)
    assert_close("pp", new_s[:, 2][~big], ref_s[:, 2][~big], rtol=2.0 ** -8, atol=1e-6)


@pytest.mark.parametrize("compat", [True, False])
@pytest.mark.parametrize("B,T,C,seed", [(2, 40, 64, 51), (3, 130, 100, 52)])
def test_bf16_backward(B, T, C, seed, compat):
    """bf16 I/O backward (wkv4-bwd-bf16, rwkv4.py:398-399): cotangents of k, v, s within a bf16 ulp plus 1e-3 of their
    rms; gw, gu (fp32 per sequence, summed over B on the host, then rounded to bf16) likewise."""
    from jaxrwkv_amd import ops
    from tests.inputs import bf16_round
    x = bf16_inputs(B, T, C, seed)
    g = np.random.default_rng(seed)
    gy = bf16_round(g.standard_normal(x["k"].shape)).astype(np.float64)
    gs = bf16_round(g.standard_normal(x["s"].shape)).astype(np.float64)
    ref_s, _ = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=compat)
    gs_eff = np.where(ref_s > -1e29, gs, 0.0)
    ref = o4.wkv4_ffi_bwd(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], gy, gs_eff, compat=compat)
    bf = torch.bfloat16
    got = ops.wkv4_bwd(dev(x["w"], bf), dev(x["u"], bf), dev(x["k"], bf), dev(x["v"], bf), dev(x["s"], bf),
                       dev(x["length"]), dev(x["new_starts"]), dev(gy, bf), dev(gs_eff, bf), compat=compat)
    torch.cuda.synchronize()
    gw, gu, gk, gv, gsi = ref
    for name, g_, rf in zip(("w", "u", "k", "v", "s"), got, (gw.sum(0), gu.sum(0), gk, gv, gsi)):
        assert_close("g" + name, host(g_), rf, rtol=2.0 ** -7, atol=1e-3, scale_atol=True)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_forward_checkpoints_equal_the_backward_own_pass(dtype):
    """hiprwkv_wkv4_fwd_ckpt + HIPRWKV_CKPT_READY: same outputs as the plain forward, and the backward that takes the
    forward's checkpoints returns bit for bit what the backward with its own checkpoint pass returns (T not a
    multiple of the 16-step segments or of the forward's 8-step blocks, resets, ragged lengths)."""
    from jaxrwkv_amd import ops
    for B, T, C, seed in [(2, 77, 100, 1), (1, 16, 64, 2), (3, 5, 65, 3), (2, 129, 128, 4)]:
        x = wkv4_inputs(B, T, C, seed=seed, p_reset=0.05, default_state=False, min_len=1)
        g = np.random.default_rng(seed)
        gy, gs = dev(g.standard_normal(x["k"].shape), dtype), dev(g.standard_normal(x["s"].shape), dtype)
        a = [dev(x[n], dtype) for n in ("w", "u", "k", "v", "s")] + [dev(x["length"]), dev(x["new_starts"])]
        plain = ops.wkv4_fwd(*a)
        new_s, y, ck = ops.wkv4_fwd(*a, want_ckpt=True)
        assert torch.equal(new_s, plain[0]) and torch.equal(y, plain[1])
        own = ops.wkv4_bwd(*a, gy, gs)
        taken = ops.wkv4_bwd(*a, gy, gs, ckpt=ck)
        for p_, q_ in zip(own, taken):
            assert torch.equal(p_, q_), (B, T, C)
