"""Randomly drawn shapes, reset densities, lengths and `compat` settings through every GPU path (chunked WKV7 and WKV6
forward and backward, the small-T kernels, WKV4 forward and backward), each checked against the float64 oracle with
the tolerances of the path's own test file.  The draw is seeded, so the cases are the same in every run."""
import numpy as np
import pytest
import torch

from oracle import wkv4 as o4, wkv6 as o6, wkv7 as o7
from tests import test_gpu_wkv4 as t4
from tests import test_gpu_wkv6_bwd_chunked as b6
from tests import test_gpu_wkv6_chunked as f6
from tests import test_gpu_wkv6_small_t as s6
from tests import test_gpu_wkv7_bwd_chunked as b7
from tests import test_gpu_wkv7_chunked as f7
from tests import test_gpu_wkv7_small_t as s7
from tests.gpu_util import assert_close
from tests.inputs import wkv4_inputs, wkv6_inputs, wkv7_inputs

pytestmark = pytest.mark.gpu


def draw_cases(n, seed):
    g = np.random.default_rng(seed)
    cases = []
    for _ in range(n):
        kind = int(g.integers(0, 4))
        if kind == 0:
            T = int(g.integers(1, 20))
        elif kind == 1:
            T = int(16 * g.integers(1, 12) + g.integers(-1, 2))      # around a chunk boundary
        elif kind == 2:
            T = int(g.integers(20, 260))
        else:
            T = int(g.integers(1, 9))                                # the small-T kernels
        cases.append(dict(B=int(g.integers(1, 4)), H=int(g.integers(1, 4)), T=T,
                          p=float(g.choice([0.0, 0.01, 0.1, 0.4])), compat=bool(g.integers(0, 2)),
                          frac=float(g.choice([0.0, 0.3, 1.0])), seed=int(g.integers(0, 1 << 30)),
                          C=int(g.choice([64, 65, 100, 128, 257])), default_state=bool(g.integers(0, 2))))
    return cases


CASES = draw_cases(48, seed=1)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{B}-T{T}-H{H}-p{p}-c{compat:d}-f{frac}".format(**c))
def test_wkv7(case):
    B, T, H, compat = case["B"], case["T"], case["H"], case["compat"]
    x = wkv7_inputs(B, T, H, 64, seed=case["seed"], bf16=True, p_reset=case["p"], min_len_frac=case["frac"])
    if case["frac"] == 0.0:
        x["length"][0] = 0
    f7.check(x, compat, *f7.run(x, compat))
    b7.check(b7.run(x, compat), b7.oracle(x, compat))
    if T <= 8:
        ref_s, ref_y = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"],
                                    x["new_starts"], compat=compat)
        new_s, y, _ = s7.run(x, torch.bfloat16, torch.float32, compat)
        assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=1e-5)
        assert_close("new_s", new_s, ref_s)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{B}-T{T}-H{H}-p{p}-c{compat:d}-f{frac}".format(**c))
def test_wkv7_fp32(case):
    """fp32 I/O: the chunked kernel on fp32 matrix instructions and the sequential kernel, both at the fp32 bar
    (rtol 1e-4, atol 1e-5), with exact zeros at the reset positions."""
    from tests import test_gpu_wkv7 as t7
    B, T, H, compat = case["B"], case["T"], case["H"], case["compat"]
    x = wkv7_inputs(B, T, H, 64, seed=case["seed"], p_reset=case["p"], min_len_frac=case["frac"])
    if case["frac"] == 0.0:
        x["length"][0] = 0
    ref_s, ref_y, ref_sa = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"],
                                        x["new_starts"], compat=compat, return_sa=True)
    for force_seq in (False, True):
        new_s, y, sa = t7.run_fwd(x, torch.float32, compat, force_seq=force_seq)
        assert_close("y", y, ref_y)
        assert_close("new_s", new_s, ref_s)
        assert_close("sa", sa, ref_sa)
        assert np.all(sa[x["new_starts"]] == 0.0)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{B}-T{T}-H{H}-p{p}-c{compat:d}-f{frac}".format(**c))
def test_wkv6(case):
    B, T, H, compat = case["B"], case["T"], case["H"], case["compat"]
    x = wkv6_inputs(B, T, H, 64, seed=case["seed"], bf16=True, p_reset=case["p"])
    if case["frac"] == 0.0:
        x["length"][0] = 0
    f6.check(x, compat, *f6.run(x, compat))
    b6.check(b6.run(x, compat), b6.oracle(x, compat))
    if T <= 8:
        ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"],
                                    compat=compat)
        new_s, y = s6.run(x, torch.bfloat16, torch.float32, compat)
        assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=1e-5)
        assert_close("new_s", new_s, ref_s)


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{B}-T{T}-C{C}-p{p}-c{compat:d}-f{frac}".format(**c))
def test_wkv4(case):
    B, T, C, compat = case["B"], case["T"], case["C"], case["compat"]
    x = wkv4_inputs(B, T, C, seed=case["seed"], p_reset=case["p"], default_state=case["default_state"], min_len=1)
    if case["frac"] == 0.0:
        x["length"][0] = 0
    ref_s, ref_y = o4.wkv4_ffi(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], compat=compat)
    new_s, y = t4.run_fwd(x, compat)
    assert_close("y", y, ref_y)
    t4.state_close(new_s, ref_s)
    g = np.random.default_rng(case["seed"])
    gy, gs = g.standard_normal(x["k"].shape), g.standard_normal(x["s"].shape)
    gs_eff = np.where(ref_s > -1e29, gs, 0.0)
    ref = o4.wkv4_ffi_bwd(x["w"], x["u"], x["k"], x["v"], x["s"], x["length"], x["new_starts"], gy, gs_eff, compat=compat)
    gw, gu, gk, gv, gsi = ref
    got = t4.run_bwd(x, gy, gs, compat)
    for name, g_, rf in zip(("w", "u", "k", "v", "s"), got, (gw.sum(0), gu.sum(0), gk, gv, gsi)):
        assert_close("g" + name, g_, rf, rtol=1e-4, atol=2e-5, scale_atol=True)
