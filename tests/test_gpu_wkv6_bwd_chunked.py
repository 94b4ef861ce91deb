"""Parity of the WKV6 backward with bf16 I/O (chunked MFMA sweeps) against the float64 oracle's vector-Jacobian
product on bf16-rounded inputs, and against the sequential fp32 sweeps on the same inputs.

Tolerances: cotangents are rounded to bf16 on output (one ulp = 2^-7 relative) plus 5e-4 of the tensor's rms for the
hi+lo bf16 operands (about 16 mantissa bits); the decay gradient is a running sum over the rest of the sequence
minus one such term and gets 1e-2 of its rms; gu is a sum over all tokens, returned in bf16; gs is fp32:
rtol 1e-4, atol 1e-4 x rms.
"""
import numpy as np
import pytest
import torch

from oracle import wkv6 as o6
from tests.gpu_util import assert_close, dev, host
from tests.inputs import wkv6_inputs

pytestmark = pytest.mark.gpu
NAMES = ("r", "k", "v", "w", "u", "s")
ATOL = dict(r=5e-4, k=5e-4, v=5e-4, w=1e-2, u=1e-3, s=1e-4)
RTOL = dict(r=2.0 ** -7, k=2.0 ** -7, v=2.0 ** -7, w=2.0 ** -7, u=2.0 ** -7, s=1e-4)


def run(x, compat, force_seq=False, with_ds=True):
    from jaxrwkv_amd import ops
    bf = torch.bfloat16
    t = {n: dev(x[n], bf) for n in ("r", "k", "v", "w", "u")}
    s, length, ns = dev(x["s"]), dev(x["length"]), dev(x["new_starts"])
    gs_out = dev(x["ds"]) if with_ds else None
    g = ops.wkv6_bwd(t["r"], t["k"], t["v"], t["w"], t["u"], s, length, ns, dev(x["dy"], bf), gs_out, compat=compat,
                     force_seq=force_seq)
    torch.cuda.synchronize()
    return dict(zip(NAMES, (host(z) for z in g)))


def oracle(x, compat, with_ds=True):
    ds = x["ds"] if with_ds else np.zeros_like(x["ds"])
    ref = o6.wkv6_bwd(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], x["dy"], ds, compat=compat)
    return dict(zip(NAMES, ref))


def check(got, ref):
    for n in NAMES:
        assert_close("g" + n, got[n], ref[n], rtol=RTOL[n], atol=ATOL[n], scale_atol=True)


@pytest.mark.parametrize("B,T,H,seed", [(1, 16, 1, 0), (2, 64, 2, 1), (1, 1, 1, 2), (2, 5, 1, 3), (1, 17, 2, 4),
                                        (2, 100, 3, 5), (1, 255, 2, 6)])
@pytest.mark.parametrize("compat", [True, False])
def test_shapes_no_resets(B, T, H, seed, compat):
    x = wkv6_inputs(B, T, H, 64, seed=seed, bf16=True, resets=False)
    check(run(x, compat), oracle(x, compat))


@pytest.mark.parametrize("seed,p", [(11, 0.05), (12, 0.2), (13, 0.5)])
@pytest.mark.parametrize("compat", [True, False])
def test_resets_inside_chunks(seed, p, compat):
    x = wkv6_inputs(2, 150, 2, 64, seed=seed, bf16=True, p_reset=p)
    x["new_starts"][0, 0] = True
    x["new_starts"][1, 15:18] = True
    x["length"][0] = 75
    x["new_starts"][0, 75] = True                    # reset exactly at `length`
    check(run(x, compat), oracle(x, compat))


@pytest.mark.parametrize("L", [0, 1, 15, 16, 17, 31, 32, 48])
def test_length_positions(L):
    x = wkv6_inputs(2, 48, 1, 64, seed=20 + L, bf16=True, p_reset=0.05)
    x["length"][:] = L
    for compat in (True, False):
        check(run(x, compat), oracle(x, compat))


def test_no_state_cotangent():
    x = wkv6_inputs(2, 80, 2, 64, seed=31, bf16=True, p_reset=0.03)
    check(run(x, True, with_ds=False), oracle(x, True, with_ds=False))


def test_matches_sequential_sweeps():
    x = wkv6_inputs(2, 512, 2, 64, seed=41, bf16=True, p_reset=1.0 / 128)
    got = run(x, True)
    seq = run(x, True, force_seq=True)
    ref = oracle(x, True)
    check(got, ref)
    check(seq, ref)
    for n in NAMES:
        assert_close("chunked-vs-sequential g" + n, got[n], seq[n], rtol=RTOL[n], atol=ATOL[n], scale_atol=True)
