"""WKV6 parity on the GPU: the HIP path (through the C ABI) against the float64 oracle and the committed fixtures."""
import os

import numpy as np
import pytest
import torch

from oracle import wkv6 as o6
from tests.gpu_util import assert_close, dev, host
from tests.inputs import wkv6_inputs

pytestmark = pytest.mark.gpu
GOLD = os.path.join(os.path.dirname(__file__), "golden", "wkv6_small.npz")
# Cotangents: rtol 1e-4 and atol 1e-5 x max(1, rms of the reference tensor).  The decay gradient is a running sum over
# the rest of the sequence of terms that cancel (er_t - k_t.(G_t v_t)), each an fp32 result: 5e-5 of its rms (measured
# up to 1.1e-5 for the chunked sweeps on fp32 matrix instructions, whose G v passes through 1/E_t, at 255 tokens).
GRAD_ATOL = dict(r=1e-5, k=1e-5, v=1e-5, w=5e-5, u=1e-5, s=1e-5)


def run_fwd(x, dtype, compat, force_seq=False):
    from jaxrwkv_amd import ops
    new_s, y = ops.wkv6_fwd(dev(x["r"], dtype), dev(x["k"], dtype), dev(x["v"], dtype), dev(x["w"], dtype),
                            dev(x["u"], dtype), dev(x["s"]), dev(x["length"]), dev(x["new_starts"]), compat=compat,
                            small_t=False, force_seq=force_seq)
    torch.cuda.synchronize()
    return host(new_s), host(y)


def run_bwd(x, dtype, compat, force_seq=False):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n], dtype).requires_grad_() for n in ("r", "k", "v", "w", "u")}
    s = dev(x["s"]).requires_grad_()
    new_s, y = ops.wkv6(t["r"], t["k"], t["v"], t["w"], t["u"], s, dev(x["length"]), dev(x["new_starts"]), compat=compat,
                        force_seq=force_seq)
    ((y.float() * dev(x["dy"])).sum() + (new_s * dev(x["ds"])).sum()).backward()
    torch.cuda.synchronize()
    return [host(t[n].grad) for n in ("r", "k", "v", "w", "u")] + [host(s.grad)]


@pytest.mark.parametrize("compat", [True, False])
def test_fp32_golden_fixture(compat):
    z = dict(np.load(GOLD))
    c = int(compat)
    new_s, y = run_fwd(z, torch.float32, compat)
    assert_close("y", y, z[f"y_c{c}"])
    assert_close("new_s", new_s, z[f"new_s_c{c}"])
    for n, g in zip("rkvwus", run_bwd(z, torch.float32, compat)):
        assert_close("g" + n, g, z[f"g{n}_c{c}"], scale_atol=True)


# fp32 I/O runs on the chunked kernel with fp32 matrix operands by default and on the sequential kernel with force_seq
@pytest.mark.parametrize("force_seq", [False, True], ids=["chunked", "seq"])
@pytest.mark.parametrize("B,T,H,seed", [(1, 1, 1, 0), (2, 17, 3, 1), (1, 33, 2, 3), (3, 100, 2, 4), (2, 257, 4, 5), (1, 1000, 1, 6)])
@pytest.mark.parametrize("compat", [True, False])
def test_fp32_forward_shapes(B, T, H, seed, compat, force_seq):
    x = wkv6_inputs(B, T, H, 64, seed=seed, p_reset=0.05)
    if T > 4:
        x["new_starts"][0, 0] = True
        x["length"][0] = T // 2
        x["new_starts"][0, T // 2] = True
    ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], compat=compat)
    new_s, y = run_fwd(x, torch.float32, compat, force_seq)
    assert_close("y", y, ref_y)
    assert_close("new_s", new_s, ref_s)


@pytest.mark.parametrize("force_seq", [False, True], ids=["chunked", "seq"])
@pytest.mark.parametrize("compat", [True, False])
@pytest.mark.parametrize("B,T,H,seed", [(2, 48, 2, 21), (1, 97, 3, 22), (1, 500, 2, 24)])
def test_fp32_backward(B, T, H, seed, compat, force_seq):
    x = wkv6_inputs(B, T, H, 64, seed=seed, p_reset=0.04)
    x["length"][0] = T // 2
    x["new_starts"][0, T // 2] = True
    ref = o6.wkv6_bwd(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"], compat=compat)
    for n, g, rf in zip("rkvwus", run_bwd(x, torch.float32, compat, force_seq), ref):
        assert_close("g" + n, g, rf, atol=GRAD_ATOL[n], scale_atol=True)


def test_length_zero():
    x = wkv6_inputs(2, 12, 1, 64, seed=23, p_reset=0.1)
    x["length"][:] = 0
    x["new_starts"][:, 0] = [True, False]
    for compat in (True, False):
        ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], compat=compat)
        new_s, y = run_fwd(x, torch.float32, compat)
        assert_close("y", y, ref_y)
        assert_close("new_s", new_s, ref_s, rtol=0, atol=0)
        ref = o6.wkv6_bwd(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"], compat=compat)
        for n, g, rf in zip("rkvwus", run_bwd(x, torch.float32, compat), ref):
            assert_close("g" + n, g, rf, scale_atol=True)


def test_bf16_io_against_float64_oracle():
    x = wkv6_inputs(2, 256, 4, 64, seed=31, bf16=True, p_reset=0.01)
    ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], compat=True)
    new_s, y = run_fwd(x, torch.bfloat16, True)        # bf16 I/O: the chunked MFMA kernel (fp16 operands)
    # tolerances of tests/test_gpu_wkv6_chunked.py
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=2e-3, scale_atol=True)
    assert_close("new_s", new_s, ref_s, rtol=1e-3, atol=2e-3, scale_atol=True)


def test_plugin_class_signature_unbatched():
    from jaxrwkv_amd.rwkv6 import HipRWKV
    x = wkv6_inputs(1, 40, 2, 64, seed=51, p_reset=0.05)
    new_s, y = HipRWKV.inner_loop(dev(x["r"][0]), dev(x["k"][0]), dev(x["v"][0]), dev(x["w"][0])[..., None],
                                  dev(x["u"])[..., None], dev(x["s"][0]), int(x["length"][0]), dev(x["new_starts"][0]))
    ref_s, ref_y = o6.wkv6_assoc_literal(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"])
    assert_close("y", host(y), ref_y[0])
    assert_close("new_s", host(new_s), ref_s[0])
