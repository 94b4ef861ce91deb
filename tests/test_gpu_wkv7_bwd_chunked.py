"""Parity of the WKV7 backward with bf16 I/O (chunked MFMA sweeps where they exist) against the float64 oracle's
vector-Jacobian product on bf16-rounded inputs, and against the sequential fp32 sweeps on the same inputs.

Tolerances: cotangents are rounded to bf16 on output (one ulp = 2^-7 relative); the chunked sweeps feed fp32
quantities to the matrix cores as bf16 hi+lo pairs (about 16 mantissa bits), so their own absolute errors are a few
1e-4 of the tensor's rms.  Two cotangents carry more.  The decay gradient is a running sum over the rest of the
sequence of O(10) terms with 2^-16 relative errors each, minus two such terms, so single elements are off by up to
1e-2 of its rms (about one bf16 ulp of a typical element).  gb_t = G_t^T sa_t is a sum with heavy cancellation (its rms
is 1/16 of the size of its terms) over the residual sa of the forward pass, which the chunked forward kernel returns
with a relative rms error of 3e-4 (fp16 operands): single elements of gb are off by up to 3.4e-3 of its rms over
these cases, ga and gr by up to 6e-4 (they see sa through the rebuilt states).  gs is fp32: rtol 1e-3, atol 1e-4 x rms.
"""
import numpy as np
import pytest
import torch

from oracle import wkv7 as o7
from tests.gpu_util import assert_close, dev, host
from tests.inputs import wkv7_inputs

pytestmark = pytest.mark.gpu
NAMES = ("r", "w", "k", "v", "a", "b", "s")
ATOL = dict(r=1e-3, w=1e-2, k=5e-4, v=5e-4, a=1e-3, b=6e-3, s=1e-4)
RTOL = dict(r=2.0 ** -7, w=2.0 ** -7, k=2.0 ** -7, v=2.0 ** -7, a=2.0 ** -7, b=2.0 ** -7, s=1e-3)


def run(x, compat, force_seq=False, with_ds=True):
    from jaxrwkv_amd import ops
    bf = torch.bfloat16
    t = {n: dev(x[n], bf) for n in ("r", "w", "k", "v", "a", "b")}
    s, length, ns = dev(x["s"]), dev(x["length"]), dev(x["new_starts"])
    new_s, y, sa = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], s, length, ns, compat=compat,
                                want_sa=True, force_seq=force_seq)
    gs_out = dev(x["ds"]) if with_ds else None
    g = ops.wkv7_bwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], s, length, ns, dev(x["dy"], bf), sa, gs_out,
                     compat=compat, force_seq=force_seq)
    torch.cuda.synchronize()
    return dict(zip(NAMES, (host(z) for z in g)))


def oracle(x, compat, with_ds=True):
    ds = x["ds"] if with_ds else np.zeros_like(x["ds"])
    ref = o7.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], x["dy"],
                      ds, compat=compat)
    return dict(zip(NAMES, ref))


def check(got, ref, names=NAMES):
    for n in names:
        assert_close("g" + n, got[n], ref[n], rtol=RTOL[n], atol=ATOL[n], scale_atol=True)


@pytest.mark.parametrize("B,T,H,seed", [(1, 16, 1, 0), (2, 64, 2, 1), (1, 1, 1, 2), (2, 5, 1, 3), (1, 17, 2, 4),
                                        (2, 100, 3, 5), (1, 255, 2, 6)])
@pytest.mark.parametrize("compat", [True, False])
def test_shapes_no_resets(B, T, H, seed, compat):
    x = wkv7_inputs(B, T, H, 64, seed=seed, bf16=True, resets=False, min_len_frac=0.3)
    check(run(x, compat), oracle(x, compat))


@pytest.mark.parametrize("seed,p", [(11, 0.05), (12, 0.2), (13, 0.5)])
@pytest.mark.parametrize("compat", [True, False])
def test_resets_inside_chunks(seed, p, compat):
    x = wkv7_inputs(2, 150, 2, 64, seed=seed, bf16=True, p_reset=p, min_len_frac=0.2)
    x["new_starts"][0, 0] = True
    x["new_starts"][1, 15:18] = True                 # chunk end, next chunk start, and the one after
    x["length"][0] = 75
    x["new_starts"][0, 75] = True                    # reset exactly at `length`
    check(run(x, compat), oracle(x, compat))


@pytest.mark.parametrize("L", [0, 1, 15, 16, 17, 31, 32, 48])
def test_length_positions(L):
    x = wkv7_inputs(2, 48, 1, 64, seed=20 + L, bf16=True, p_reset=0.05)
    x["length"][:] = L
    for compat in (True, False):
        check(run(x, compat), oracle(x, compat))


def test_no_state_cotangent():
    x = wkv7_inputs(2, 80, 2, 64, seed=31, bf16=True, p_reset=0.03)
    check(run(x, True, with_ds=False), oracle(x, True, with_ds=False))


def test_matches_sequential_sweeps():
    x = wkv7_inputs(2, 512, 2, 64, seed=41, bf16=True, p_reset=1.0 / 128)
    got = run(x, True)
    seq = run(x, True, force_seq=True)
    ref = oracle(x, True)
    check(got, ref)
    check(seq, ref)
    for n in NAMES:
        assert_close("chunked-vs-sequential g" + n, got[n], seq[n], rtol=RTOL[n], atol=ATOL[n], scale_atol=True)


@pytest.mark.parametrize("shift", [-40, -17, 12, 30])
def test_cotangents_scale_by_powers_of_two_exactly(shift):
    """The workspace between the sweeps is 16-bit fixed point with a power-of-two scale per 16 x 16 tile, chosen from
    the tile's largest magnitude; every other step is fp32 arithmetic or a bf16 pair.  Multiplying dy and the state
    cotangent by 2^shift must therefore multiply every cotangent by 2^shift to the bit (as long as nothing leaves the
    normal range): gradients 1e-12 or 1e9 times the usual size keep their 16 bits."""
    x = wkv7_inputs(2, 150, 2, 64, seed=61, bf16=True, p_reset=0.03, min_len_frac=0.4)
    base = run(x, True)
    c = 2.0 ** shift
    y = dict(x)
    y["dy"], y["ds"] = x["dy"] * c, x["ds"] * c
    scaled = run(y, True)
    for n in NAMES:
        assert np.array_equal(scaled[n], base[n] * c), n


def test_a_non_finite_cotangent_stays_visible():
    """A tile of the workspace that holds inf or NaN is marked as a whole, so the sweeps that read it cannot turn a
    non-finite value into a finite one."""
    x = wkv7_inputs(1, 64, 1, 64, seed=62, bf16=True, resets=False)
    x["length"][:] = 64
    for bad in (np.inf, np.nan):
        y = dict(x)
        y["dy"] = x["dy"].copy()
        y["dy"][0, 37, 0, 5] = bad
        g = run(y, True)
        for n in ("r", "k", "a", "b", "w"):
            assert not np.all(np.isfinite(g[n][0, :38])), (bad, n)
