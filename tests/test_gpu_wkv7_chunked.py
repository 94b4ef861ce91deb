"""Parity of the chunked MFMA WKV7 forward (the bf16 I/O path) against the float64 oracle on bf16-rounded inputs.

Tolerances: the kernel feeds the matrix cores fp16 operands (11 significant bits; bf16 hi+lo pairs in the Gram tiles)
and keeps the carried state in fp32, which is what the bf16 bar (TVD of projected outputs < 1e-3, checked on a longer
sequence) needs and no more: tests/precision_model.py predicts relative rms errors of 2e-4 for y before its rounding,
1-2e-4 for the final state and 3e-4 for sa, and the kernel measures the same.  Element-wise that is: y within one
bf16 ulp of the oracle plus 2e-3 of its rms, the fp32 state within 1e-3 relative plus 2e-3 of its rms (half a bf16
ulp of a typical element: the reference returns a bf16 state for bf16 inputs, rwkv7.py:346), sa within 2e-3 relative
plus 3e-3 of its rms.  Largest values seen over these cases and the random-shape cases: 1.1e-3, 1.3e-3, 1.4e-3.
"""
import numpy as np
import pytest
import torch

from oracle import wkv7 as o7
from tests.gpu_util import assert_close, dev, host, tvd_of_projected
from tests.inputs import bf16_round, wkv7_inputs

pytestmark = pytest.mark.gpu
Y_ATOL, S_RTOL, S_ATOL, SA_RTOL, SA_ATOL = 2e-3, 1e-3, 2e-3, 2e-3, 3e-3      # atol in units of the tensor's rms


def run(x, compat, state_dtype=torch.float32, force_seq=False, want_sa=True):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n], torch.bfloat16) for n in ("r", "w", "k", "v", "a", "b")}
    new_s, y, sa = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"], state_dtype),
                                dev(x["length"]), dev(x["new_starts"]), compat=compat, want_sa=want_sa,
                                force_seq=force_seq, small_t=False)
    torch.cuda.synchronize()
    return host(new_s), host(y), (host(sa) if sa is not None else None)


def check(x, compat, new_s, y, sa):
    ref_s, ref_y, ref_sa = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"],
                                        x["new_starts"], compat=compat, return_sa=True)
    assert_close("new_s", new_s, ref_s, rtol=S_RTOL, atol=S_ATOL, scale_atol=True)
    if sa is not None:
        assert_close("sa", sa, ref_sa, rtol=SA_RTOL, atol=SA_ATOL, scale_atol=True)
        assert np.all(sa[x["new_starts"]] == 0.0)        # state entering a reset token is exactly zero
    # y is bf16 on output: within one bf16 ulp (2^-7 relative) of the oracle, plus the operand-precision slack above
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=Y_ATOL, scale_atol=True)
    if compat:
        nxt = np.zeros_like(x["new_starts"])
        nxt[:, :-1] = x["new_starts"][:, 1:]
        assert np.all(y[nxt] == 0.0)
    return ref_s, ref_y


@pytest.mark.parametrize("B,T,H,seed", [(1, 16, 1, 0), (2, 64, 2, 1), (1, 1, 1, 2), (2, 5, 1, 3), (1, 17, 2, 4),
                                        (2, 100, 3, 5), (1, 255, 2, 6), (2, 513, 2, 7)])
@pytest.mark.parametrize("compat", [True, False])
def test_shapes_no_resets(B, T, H, seed, compat):
    x = wkv7_inputs(B, T, H, 64, seed=seed, bf16=True, resets=False, min_len_frac=0.3)
    check(x, compat, *run(x, compat))


@pytest.mark.parametrize("seed,p", [(11, 0.05), (12, 0.2), (13, 0.5)])
@pytest.mark.parametrize("compat", [True, False])
def test_resets_inside_chunks(seed, p, compat):
    x = wkv7_inputs(2, 150, 2, 64, seed=seed, bf16=True, p_reset=p, min_len_frac=0.2)
    x["new_starts"][0, 0] = True
    x["new_starts"][1, 15:18] = True                 # chunk end, next chunk start, and the one after
    x["length"][0] = 75
    x["new_starts"][0, 75] = True                    # reset exactly at `length`
    check(x, compat, *run(x, compat))


@pytest.mark.parametrize("L", [0, 1, 15, 16, 17, 31, 32, 48])
def test_length_positions(L):
    x = wkv7_inputs(2, 48, 1, 64, seed=20 + L, bf16=True, p_reset=0.05)
    x["length"][:] = L
    for compat in (True, False):
        new_s, y, sa = run(x, compat)
        check(x, compat, new_s, y, sa)


def test_bf16_state_dtype_and_no_sa():
    x = wkv7_inputs(2, 80, 2, 64, seed=31, bf16=True, p_reset=0.03)
    x["s"] = bf16_round(x["s"]).astype(np.float64)
    new_s, y, sa = run(x, True, state_dtype=torch.bfloat16, want_sa=False)
    ref_s, ref_y = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], compat=True)
    assert sa is None
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=Y_ATOL, scale_atol=True)
    assert_close("new_s", new_s, ref_s, rtol=2.0 ** -7, atol=S_ATOL, scale_atol=True)


@pytest.mark.parametrize("B,T,H,seed,p", [(1, 16, 1, 50, 0.0), (2, 17, 2, 51, 0.1), (1, 159, 2, 52, 0.05),
                                          (2, 160, 1, 53, 0.0), (1, 161, 3, 54, 0.02), (2, 333, 2, 55, 0.01),
                                          (1, 9, 1, 56, 0.2), (1, 1000, 2, 57, 0.004)])
def test_the_two_instantiations_agree_bit_for_bit(B, T, H, seed, p):
    """The launch without `sa` (consumers store y) and the one with it (y parked in LDS, written out by the producers,
    the last slots by extra steps after the last chunk) must give the same bits; the first is also held to the oracle
    here, the second by every other test of this file."""
    x = wkv7_inputs(B, T, H, 64, seed=seed, bf16=True, p_reset=p, min_len_frac=0.3)
    for compat in (True, False):
        s0, y0, none = run(x, compat, want_sa=False)
        s1, y1, sa1 = run(x, compat, want_sa=True)
        assert none is None
        assert np.array_equal(y0, y1) and np.array_equal(s0, s1)
        check(x, compat, s0, y0, None)


def test_matches_sequential_kernel_and_tvd_bar():
    x = wkv7_inputs(2, 1024, 4, 64, seed=41, bf16=True, p_reset=1.0 / 256)
    new_s, y, sa = run(x, True)
    ref_s, ref_y = check(x, True, new_s, y, sa)
    s2, y2, sa2 = run(x, True, force_seq=True)
    assert_close("seq-vs-chunk new_s", new_s, s2, rtol=S_RTOL, atol=S_ATOL, scale_atol=True)
    assert_close("seq-vs-chunk sa", sa, sa2, rtol=SA_RTOL, atol=SA_ATOL, scale_atol=True)
    # the bf16 bar: total-variation distance of projected, group-normed outputs below 1e-3
    tvd = tvd_of_projected(y, bf16_round(ref_y).astype(np.float64))
    assert tvd.max() < 1e-3, tvd.max()
    tvd_unrounded = tvd_of_projected(y, ref_y)
    tvd_floor = tvd_of_projected(bf16_round(ref_y).astype(np.float64), ref_y)    # cost of the bf16 output alone
    assert tvd_unrounded.max() < tvd_floor.max() + 5e-4, (tvd_unrounded.max(), tvd_floor.max())


def test_strong_decay_is_finite_and_counted():
    """A key channel whose log decay over a 16-token chunk is below -80 gets that chunk's steps scaled to -80 in
    total: finite, inexact, and counted by hiprwkv_numeric_events.  Decays above the floor are exact and silent."""
    from jaxrwkv_amd import ops
    x = wkv7_inputs(1, 64, 1, 64, seed=51, bf16=True, resets=False, lengths=False)
    x["w"] = bf16_round(np.clip(x["w"] + 1.5, None, 1.6)).astype(np.float64)    # exp(1.6) * 16 = 79.2 < 80
    before = ops.numeric_events()
    new_s, y, sa = run(x, False)
    check(x, False, new_s, y, sa)
    assert ops.numeric_events() == before                  # no chunk reached the floor
    x["w"][:] = 4.0                                         # exp(4) * 16 = 874: every chunk of every channel
    new_s, y, sa = run(x, False)
    assert np.all(np.isfinite(y)) and np.all(np.isfinite(new_s))
    assert ops.numeric_events() >= before + 4 * 2           # four chunks, two 32-key halves each
    # the fp32-I/O chunked kernel has the same floor and counts the same way
    before = ops.numeric_events()
    t = {n: dev(x[n]) for n in "rwkvab"}
    s32, y32, _ = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"]), small_t=False)
    assert bool(torch.isfinite(y32).all()) and ops.numeric_events() >= before + 4 * 2
    # the sequential kernels have no floor: nothing is counted there
    before = ops.numeric_events()
    ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"]), small_t=False, force_seq=True)
    assert ops.numeric_events() == before


def test_values_beyond_the_fp16_range_give_inf_and_are_counted():
    """The bf16 forward feeds IEEE-half operands to the matrix cores: v (and with it the state) beyond 65504 cannot
    be represented.  The conversion overflows to infinity, so y and the state come back non-finite from that token
    on, and hiprwkv_numeric_events advances; the sequential kernel (HIPRWKV_FORCE_SEQ) has no such limit and still
    matches the oracle."""
    from jaxrwkv_amd import ops
    x = wkv7_inputs(1, 64, 1, 64, seed=77, bf16=True, resets=False, lengths=False)
    x["v"] = bf16_round(x["v"] * 1.0e5).astype(np.float64)
    t = {n: dev(x[n], torch.bfloat16) for n in "rwkvab"}
    before = ops.numeric_events()
    _, y, _ = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"]), small_t=False)
    assert not bool(torch.isfinite(y.float()).all())
    assert ops.numeric_events() > before
    before = ops.numeric_events()
    new_s, y, _ = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"]), small_t=False, force_seq=True)
    assert ops.numeric_events() == before
    ref_s, ref_y = o7.wkv7_base(*[x[n] for n in "rwkvab"], x["s"], x["length"], x["new_starts"], compat=True)
    assert_close("y", host(y), ref_y, rtol=2.0 ** -7, atol=1e-4, scale_atol=True)
    assert_close("new_s", host(new_s), ref_s, rtol=1e-4, atol=1e-4, scale_atol=True)


@pytest.mark.parametrize("scale", [1.0e-3, 64.0])
def test_magnitudes_inside_the_documented_range_keep_the_tolerances(scale):
    """v and the state scaled by 1e-3 or 64: the IEEE-half operands still hold 11 significant bits there, and y, the
    state and sa stay within the tolerances of the unscaled case (the op is linear in (v, s))."""
    x = wkv7_inputs(2, 150, 2, 64, seed=83, bf16=True, p_reset=0.02)
    x["v"] = bf16_round(x["v"] * scale).astype(np.float64)
    x["s"] = (x["s"] * scale).astype(np.float32).astype(np.float64)
    new_s, y, sa = run(x, True)
    check(x, True, new_s, y, sa)
