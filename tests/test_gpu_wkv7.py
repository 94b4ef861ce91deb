"""WKV7 parity on the GPU: the HIP path (through the C ABI) against the float64 oracle and the committed fixtures."""
import os

import numpy as np
import pytest
import torch

from oracle import wkv7 as o7
from tests.gpu_util import assert_close, dev, host, tvd_of_projected
from tests.inputs import bf16_round, wkv7_inputs

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "wkv7_small.npz")
# Cotangents: rtol 1e-4 and atol 1e-5 x max(1, rms of the reference tensor).  The decay gradient is obtained in
# fp32 from the cancellation D_t - k.dk - b.db of O(10) terms, so its absolute error is a few 1e-5 of its rms.
GRAD_ATOL = dict(r=1e-5, w=5e-5, k=1e-5, v=1e-5, a=1e-5, b=1e-5, s=1e-5)


def run_fwd(x, dtype, compat, state_dtype=torch.float32, force_seq=False):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n], dtype) for n in ("r", "w", "k", "v", "a", "b")}
    new_s, y, sa = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"], state_dtype),
                                dev(x["length"]), dev(x["new_starts"]), compat=compat, want_sa=True, small_t=False,
                                force_seq=force_seq)
    torch.cuda.synchronize()
    return host(new_s), host(y), host(sa)


def run_bwd(x, dtype, compat, force_seq=False):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n], dtype).requires_grad_() for n in ("r", "w", "k", "v", "a", "b")}
    s = dev(x["s"]).requires_grad_()
    new_s, y = ops.wkv7(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], s, dev(x["length"]), dev(x["new_starts"]), compat=compat,
                        force_seq=force_seq)
    loss = (y.float() * dev(x["dy"])).sum() + (new_s * dev(x["ds"])).sum()
    loss.backward()
    torch.cuda.synchronize()
    return [host(t[n].grad) for n in ("r", "w", "k", "v", "a", "b")] + [host(s.grad)]


@pytest.mark.parametrize("compat", [True, False])
def test_fp32_golden_fixture(compat):
    z = dict(np.load(GOLD))
    c = int(compat)
    new_s, y, _ = run_fwd(z, torch.float32, compat)
    assert_close("y", y, z[f"y_c{c}"])
    assert_close("new_s", new_s, z[f"new_s_c{c}"])
    x = dict(z)
    x["dy"], x["ds"] = z["dy"], z["ds"]
    grads = run_bwd(x, torch.float32, compat)
    for n, g in zip("rwkvabs", grads):
        assert_close("g" + n, g, z[f"g{n}_c{c}"], atol=GRAD_ATOL[n], scale_atol=True)


@pytest.mark.parametrize("B,T,H,seed", [(1, 1, 1, 0), (2, 17, 3, 1), (2, 32, 2, 2), (1, 33, 2, 3), (3, 100, 2, 4), (2, 257, 4, 5)])
@pytest.mark.parametrize("compat", [True, False])
def test_fp32_forward_shapes(B, T, H, seed, compat):
    x = wkv7_inputs(B, T, H, 64, seed=seed, p_reset=0.05, min_len_frac=0.3)
    if T > 4:
        x["new_starts"][0, 0] = True                     # reset at the very first token
        x["length"][0] = T // 2
        x["new_starts"][0, T // 2] = True                # reset exactly at `length` (Q2)
    ref_s, ref_y, ref_sa = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"],
                                        x["new_starts"], compat=compat, return_sa=True)
    new_s, y, sa = run_fwd(x, torch.float32, compat)
    assert_close("y", y, ref_y)
    assert_close("new_s", new_s, ref_s)
    assert_close("sa", sa, ref_sa)
    # exactly equal reset positions: the state entering a reset token is zero, so sa is exactly 0 there
    assert np.all(sa[x["new_starts"]] == 0.0)
    if compat:
        nxt = np.zeros_like(x["new_starts"])
        nxt[:, :-1] = x["new_starts"][:, 1:]
        assert np.all(y[nxt] == 0.0)


def test_length_zero_and_none():
    from jaxrwkv_amd import ops
    x = wkv7_inputs(2, 20, 2, 64, seed=9, p_reset=0.1)
    x["length"][:] = 0
    x["new_starts"][:, 0] = [True, False]
    for compat in (True, False):
        ref_s, ref_y = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], compat=compat)
        new_s, y, _ = run_fwd(x, torch.float32, compat)
        assert_close("y", y, ref_y)
        assert_close("new_s", new_s, ref_s, rtol=0, atol=0)
    # defaults of llm.py:78-81: length = T, no resets
    t = {n: dev(x[n]) for n in ("r", "w", "k", "v", "a", "b")}
    new_s, y, _ = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"]))
    ref_s, ref_y = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"])
    assert_close("y", host(y), ref_y)
    assert_close("new_s", host(new_s), ref_s)


# fp32 I/O runs on the chunked kernels with fp32 matrix operands by default and on the sequential kernels with
# force_seq: both are held to the same bar against the float64 oracle.
@pytest.mark.parametrize("force_seq", [False, True], ids=["chunked", "seq"])
@pytest.mark.parametrize("compat", [True, False])
@pytest.mark.parametrize("B,T,H,seed", [(2, 48, 2, 21), (1, 97, 3, 22)])
def test_fp32_backward(B, T, H, seed, compat, force_seq):
    x = wkv7_inputs(B, T, H, 64, seed=seed, p_reset=0.04, min_len_frac=0.4)
    x["length"][0] = T // 2
    x["new_starts"][0, T // 2] = True
    ref = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"], compat=compat)
    got = run_bwd(x, torch.float32, compat, force_seq)
    for n, g, rf in zip("rwkvabs", got, ref):
        assert_close("g" + n, g, rf, atol=GRAD_ATOL[n], scale_atol=True)


@pytest.mark.parametrize("force_seq", [False, True], ids=["chunked", "seq"])
def test_backward_length_zero(force_seq):
    x = wkv7_inputs(2, 12, 1, 64, seed=23, p_reset=0.1)
    x["length"][:] = 0
    for compat in (True, False):
        ref = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"], compat=compat)
        got = run_bwd(x, torch.float32, compat, force_seq)
        for n, g, rf in zip("rwkvabs", got, ref):
            assert_close("g" + n, g, rf, atol=GRAD_ATOL[n], scale_atol=True)


@pytest.mark.parametrize("B,T,H,p,seed", [(1, 640, 2, 0.0, 31), (1, 1100, 1, 0.004, 32), (2, 333, 2, 0.02, 33), (1, 2048, 1, 0.0, 35)])
def test_fp32_backward_long(B, T, H, p, seed):
    """Hundreds of chunks: the carried cotangent, the running sum of the decay gradient and the records handed from the
    forward sweep to the last one, all in fp32 against the float64 oracle; the length of one sequence ends inside a
    chunk, with a reset right after it.  The decay gradient at token t is a sum over every later token of the segment
    of terms that cancel, each an fp32 result: its error grows with the distance to the end.  Measured at 640-2048
    tokens without resets: 2.0-2.55 times the bound of the short cases for these kernels and 1.8-2.05 times for the
    sequential ones (a compensated carry changes nothing: the terms' own rounding is what adds up), so gw is held to
    2e-4 of its rms here and the other cotangents to the bound of the short cases."""
    x = wkv7_inputs(B, T, H, 64, seed=seed, p_reset=p, min_len_frac=0.6)
    x["length"][0] = T - 37
    x["new_starts"][0, T - 37] = True
    ref = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"], compat=True)
    got = run_bwd(x, torch.float32, True)
    for n, g, rf in zip("rwkvabs", got, ref):
        assert_close("g" + n, g, rf, atol=2e-4 if n == "w" else GRAD_ATOL[n], scale_atol=True)


def test_fp32_backward_with_bf16_state():
    """fp32 token tensors with a bf16 state and state cotangent (the state dtype is independent of the I/O dtype)."""
    from jaxrwkv_amd import ops
    x = wkv7_inputs(2, 50, 2, 64, seed=34, p_reset=0.03, min_len_frac=0.5)
    x["s"], x["ds"] = bf16_round(x["s"]), bf16_round(x["ds"])
    ref = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"], compat=True)
    t = [dev(x[n], torch.float32) for n in ("r", "w", "k", "v", "a", "b")]
    s, ln, ns = dev(x["s"], torch.bfloat16), dev(x["length"]), dev(x["new_starts"])
    _, _, sa = ops.wkv7_fwd(*t, s, ln, ns, compat=True, want_sa=True, small_t=False)
    got = ops.wkv7_bwd(*t, s, ln, ns, dev(x["dy"], torch.float32), sa, dev(x["ds"], torch.bfloat16), compat=True)
    torch.cuda.synchronize()
    for n, g, rf in zip("rwkvab", got[:6], ref[:6]):
        assert_close("g" + n, host(g), rf, atol=GRAD_ATOL[n], scale_atol=True)
    assert_close("gs", host(got[6].float()), ref[6], rtol=2.0 ** -7, atol=1e-5)


def test_bf16_io_against_float64_oracle():
    x = wkv7_inputs(2, 256, 4, 64, seed=31, bf16=True, p_reset=0.01)
    ref_s, ref_y = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], compat=True)
    new_s, y, _ = run_fwd(x, torch.bfloat16, True)
    # y is rounded to bf16 on output: half an ulp = 2^-9 relative
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=2e-3, scale_atol=True)
    # fp32 state out of the chunked MFMA kernel (fp16 operands, 11 significant bits: see test_gpu_wkv7_chunked.py)
    assert_close("new_s", new_s, ref_s, rtol=1e-3, atol=2e-3, scale_atol=True)
    # bf16 bar: TVD of projected outputs below 1e-3, against the oracle's y rounded to the same output type
    tvd = tvd_of_projected(y, bf16_round(ref_y).astype(np.float64))
    assert tvd.max() < 1e-3, tvd.max()


def test_split_call_equals_single_call_and_batch_independence():
    x = wkv7_inputs(2, 64, 2, 64, seed=41, resets=False, lengths=False)
    s_full, y_full, _ = run_fwd(x, torch.float32, False)
    cut = 37
    xa = {n: (x[n][:, :cut] if n in "rwkvab" else x[n]) for n in x}
    xa["length"] = np.full(2, cut, np.int32); xa["new_starts"] = x["new_starts"][:, :cut]
    s_a, y_a, _ = run_fwd(xa, torch.float32, False)
    xb = {n: (x[n][:, cut:] if n in "rwkvab" else x[n]) for n in x}
    xb["s"] = s_a; xb["length"] = np.full(2, 64 - cut, np.int32); xb["new_starts"] = x["new_starts"][:, cut:]
    s_b, y_b, _ = run_fwd(xb, torch.float32, False)
    assert_close("y", np.concatenate([y_a, y_b], 1), y_full)
    assert_close("s", s_b, s_full)
    x1 = {n: x[n][1:] for n in x}
    s_1, y_1, _ = run_fwd(x1, torch.float32, False)
    assert np.array_equal(y_1, y_full[1:]) and np.array_equal(s_1, s_full[1:])


def test_plugin_class_signature_unbatched():
    from jaxrwkv_amd.rwkv7 import HipRWKV
    x = wkv7_inputs(1, 40, 2, 64, seed=51, p_reset=0.05)
    args = [dev(x[n][0]) for n in ("r", "w", "k", "v", "a", "b", "s")]
    new_s, y = HipRWKV.inner_loop(*args, int(x["length"][0]), dev(x["new_starts"][0]))
    ref_s, ref_y = o7.wkv7_assoc_literal(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"])
    assert y.shape == (40, 2, 64) and new_s.shape == (2, 64, 64)
    assert_close("y", host(y), ref_y[0])
    assert_close("new_s", host(new_s), ref_s[0])
