"""Parity of the chunked MFMA WKV6 forward (the bf16 I/O path) against the float64 oracle on bf16-rounded inputs.

Tolerances.  The kernel (jaxrwkv_amd/csrc/wkv6_fwd.hip) feeds the matrix cores fp16 operands (11 significant bits:
the state, qt, ke, v; the Gram tile as an fp16 pair, its operands as bf16 pairs), so y before its bf16 rounding and the
fp32 state carry relative errors of a few 1e-4 of their rms.  A scan of every case of this file and of
tests/test_gpu_random_shapes.py found, in units of the compared array's rms, at most 1.2e-3 for y beyond one bf16 ulp
of the oracle's value and 1.3e-3 for the state beyond 1e-3 of its own magnitude; the figures below leave a factor
1.5 on top.  The bf16 bar proper (TVD of projected outputs < 1e-3) is checked on a longer sequence.
"""
import numpy as np
import pytest
import torch

from oracle import wkv6 as o6
from tests.gpu_util import assert_close, dev, host, tvd_of_projected
from tests.inputs import bf16_round, wkv6_inputs

pytestmark = pytest.mark.gpu
Y_ATOL, S_RTOL, S_ATOL = 2e-3, 1e-3, 2e-3      # atol in units of the reference array's rms


def run(x, compat, state_dtype=torch.float32, force_seq=False):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n], torch.bfloat16) for n in ("r", "k", "v", "w", "u")}
    new_s, y = ops.wkv6_fwd(t["r"], t["k"], t["v"], t["w"], t["u"], dev(x["s"], state_dtype), dev(x["length"]),
                            dev(x["new_starts"]), compat=compat, force_seq=force_seq, small_t=False)
    torch.cuda.synchronize()
    return host(new_s), host(y)


def check(x, compat, new_s, y):
    ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"],
                                compat=compat)
    assert_close("new_s", new_s, ref_s, rtol=S_RTOL, atol=S_ATOL, scale_atol=True)
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=Y_ATOL, scale_atol=True)
    return ref_s, ref_y


@pytest.mark.parametrize("B,T,H,seed", [(1, 16, 1, 0), (2, 64, 2, 1), (1, 1, 1, 2), (2, 5, 1, 3), (1, 17, 2, 4),
                                        (2, 100, 3, 5), (1, 255, 2, 6), (2, 513, 2, 7)])
@pytest.mark.parametrize("compat", [True, False])
def test_shapes_no_resets(B, T, H, seed, compat):
    x = wkv6_inputs(B, T, H, 64, seed=seed, bf16=True, resets=False)
    check(x, compat, *run(x, compat))


@pytest.mark.parametrize("seed,p", [(11, 0.05), (12, 0.2), (13, 0.5)])
@pytest.mark.parametrize("compat", [True, False])
def test_resets_inside_chunks(seed, p, compat):
    x = wkv6_inputs(2, 150, 2, 64, seed=seed, bf16=True, p_reset=p)
    x["new_starts"][0, 0] = True
    x["new_starts"][1, 15:18] = True                 # chunk end, next chunk start, and the one after
    x["length"][0] = 75
    x["new_starts"][0, 75] = True                    # reset exactly at `length`
    check(x, compat, *run(x, compat))


@pytest.mark.parametrize("L", [0, 1, 15, 16, 17, 31, 32, 48])
def test_length_positions(L):
    x = wkv6_inputs(2, 48, 1, 64, seed=20 + L, bf16=True, p_reset=0.05)
    x["length"][:] = L
    for compat in (True, False):
        check(x, compat, *run(x, compat))


def test_bf16_state_dtype():
    x = wkv6_inputs(2, 80, 2, 64, seed=31, bf16=True, p_reset=0.03)
    x["s"] = bf16_round(x["s"]).astype(np.float64)
    new_s, y = run(x, True, state_dtype=torch.bfloat16)
    ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], compat=True)
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=Y_ATOL, scale_atol=True)
    assert_close("new_s", new_s, ref_s, rtol=2.0 ** -7, atol=S_ATOL, scale_atol=True)


def test_matches_sequential_kernel_and_tvd_bar():
    x = wkv6_inputs(2, 1024, 4, 64, seed=41, bf16=True, p_reset=1.0 / 256)
    new_s, y = run(x, True)
    ref_s, ref_y = check(x, True, new_s, y)
    s2, y2 = run(x, True, force_seq=True)
    assert_close("seq-vs-chunk new_s", new_s, s2, rtol=S_RTOL, atol=S_ATOL, scale_atol=True)
    assert_close("seq-vs-chunk y", y, y2, rtol=2.0 ** -7, atol=Y_ATOL, scale_atol=True)
    # the bf16 bar: total-variation distance of projected, group-normed outputs below 1e-3
    tvd = tvd_of_projected(y, bf16_round(ref_y).astype(np.float64))
    assert tvd.max() < 1e-3, tvd.max()
    tvd_unrounded = tvd_of_projected(y, ref_y)
    tvd_floor = tvd_of_projected(bf16_round(ref_y).astype(np.float64), ref_y)    # cost of the bf16 output alone
    assert tvd_unrounded.max() < tvd_floor.max() + 5e-4, (tvd_unrounded.max(), tvd_floor.max())


def test_strong_decay_is_finite():
    # decays far below the clamp must not produce inf/nan; down to e^-4 per token the result matches the oracle
    x = wkv6_inputs(1, 64, 1, 64, seed=51, bf16=True, resets=False, lengths=False)
    x["w"] = bf16_round(np.clip(x["w"] * 3.0, -4.0, None)).astype(np.float64)
    check(x, False, *run(x, False))
    x["w"][:] = -50.0
    new_s, y = run(x, False)
    assert np.all(np.isfinite(y)) and np.all(np.isfinite(new_s))
