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
    """fp32 I/O: the chunked kernels on fp32 matrix instructions and the sequential kernels, forward and backward, both
    at the fp32 bar (rtol 1e-4, atol 1e-5; cotangents in units of their rms), with exact zeros at the reset positions."""
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
    ref = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], x["dy"],
                      x["ds"], compat=compat)
    for force_seq in (False, True):      # the three sweeps on fp32 matrix instructions, and the sequential ones
        got = t7.run_bwd(x, torch.float32, compat, force_seq)
        for n, g, rf in zip("rwkvabs", got, ref):
            assert_close("g" + n, g, rf, atol=t7.GRAD_ATOL[n], scale_atol=True)


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


@pytest.mark.parametrize("case", CASES, ids=lambda c: "B{B}-T{T}-H{H}-p{p}-c{compat:d}-f{frac}".format(**c))
def test_wkv6_fp32(case):
    """fp32 I/O: the chunked kernels on fp32 matrix instructions and the sequential ones, forward and backward, at the
    fp32 bar."""
    from tests import test_gpu_wkv6 as t6
    B, T, H, compat = case["B"], case["T"], case["H"], case["compat"]
    x = wkv6_inputs(B, T, H, 64, seed=case["seed"], p_reset=case["p"])
    if case["frac"] == 0.0:
        x["length"][0] = 0
    ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"],
                                compat=compat)
    for force_seq in (False, True):
        new_s, y = t6.run_fwd(x, torch.float32, compat, force_seq)
        assert_close("y", y, ref_y)
        assert_close("new_s", new_s, ref_s)
    ref = o6.wkv6_bwd(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], x["dy"], x["ds"],
                      compat=compat)
    for force_seq in (False, True):      # the two sweeps on fp32 matrix instructions, and the sequential kernel
        for n, g, rf in zip("rkvwus", t6.run_bwd(x, torch.float32, compat, force_seq), ref):
            assert_close("g" + n, g, rf, atol=t6.GRAD_ATOL[n], scale_atol=True)


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


# ---------------------------------------------------------------------------------------------------- long sequences
# Sequences of 300-1500 tokens.  The forward checks are the element-wise ones of the short cases.  The bf16 backward is
# held to a bound in two parts, in units of each cotangent's rms and after one bf16 ulp of the reference (rtol 2^-7)
# has been taken off: the 99.99th percentile of the absolute error stays within 0.6 of the tolerance of the short cases
# (b7.ATOL; measured 0.01-0.36 over these cases), and the largest single element within twice that tolerance (measured
# 0.01-0.73 here; a draw of 1500 other cases had ten single elements between 1.01 and 1.24).  A running sum over the rest of the sequence (the decay
# gradient) and the sums with cancellation behind ga and gb leave a thin tail of single elements beyond the
# element-wise figure once a sequence is more than a thousand tokens long; the two-part bound states how thin.
LONG_CASES = [dict(B=2, T=300, H=2, p=0.0, compat=True, seed=101), dict(B=1, T=511, H=2, p=0.01, compat=False, seed=102),
              dict(B=1, T=640, H=3, p=0.0, compat=True, seed=103), dict(B=2, T=777, H=1, p=0.01, compat=True, seed=104),
              dict(B=1, T=1024, H=2, p=0.002, compat=False, seed=105), dict(B=1, T=1100, H=2, p=0.0, compat=True, seed=106),
              dict(B=1, T=1333, H=1, p=0.01, compat=True, seed=107), dict(B=1, T=1500, H=2, p=0.002, compat=True, seed=108)]
TAIL_Q, TAIL_Q_LIMIT, TAIL_MAX = 0.9999, 0.6, 2.0


def tail_check(got, ref, names=b7.NAMES):
    worst = {}
    for n in names:
        g, r = np.asarray(got[n], np.float64), np.asarray(ref[n], np.float64)
        rms = max(1.0, float(np.sqrt(np.mean(r ** 2))))
        excess = np.maximum(np.abs(g - r) - b7.RTOL[n] * np.abs(r), 0.0) / (b7.ATOL[n] * rms)
        q, m = float(np.quantile(excess, TAIL_Q)), float(excess.max())
        worst[n] = (q, m)
        assert q <= TAIL_Q_LIMIT, f"g{n}: the {TAIL_Q} quantile of the error is {q:.2f} of the tolerance (limit {TAIL_Q_LIMIT})"
        assert m <= TAIL_MAX, f"g{n}: the largest error is {m:.2f} of the tolerance (limit {TAIL_MAX})"
    return worst


@pytest.mark.parametrize("case", LONG_CASES, ids=lambda c: "B{B}-T{T}-H{H}-p{p}-c{compat:d}".format(**c))
def test_wkv7_long(case):
    x = wkv7_inputs(case["B"], case["T"], case["H"], 64, seed=case["seed"], bf16=True, p_reset=case["p"], min_len_frac=0.7)
    f7.check(x, case["compat"], *f7.run(x, case["compat"]))
    worst = tail_check(b7.run(x, case["compat"]), b7.oracle(x, case["compat"]))
    print("T=%d" % case["T"], " ".join("g%s %.2f/%.2f" % (n, q, m) for n, (q, m) in worst.items()))
