"""The small-T (decode) WKV6 kernel, T = 1..8, against the float64 oracle: fp32 arithmetic, so the fp32 bar
(rtol 1e-4 / atol 1e-5) applies to fp32 I/O; with bf16 I/O y is within one bf16 ulp and a bf16 state within one ulp."""
import numpy as np
import pytest
import torch

from oracle import wkv6 as o6
from tests.gpu_util import assert_close, dev, host
from tests.inputs import bf16_round, wkv6_inputs

pytestmark = pytest.mark.gpu


def run(x, io, st, compat, small_t=True):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n], io) for n in ("r", "k", "v", "w", "u")}
    new_s, y = ops.wkv6_fwd(t["r"], t["k"], t["v"], t["w"], t["u"], dev(x["s"], st), dev(x["length"]),
                            dev(x["new_starts"]), compat=compat, small_t=small_t)
    torch.cuda.synchronize()
    return host(new_s), host(y)


@pytest.mark.parametrize("T", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("compat", [True, False])
def test_fp32(T, compat):
    x = wkv6_inputs(3, T, 2, 64, seed=100 + T, p_reset=0.3)
    x["length"][0] = 0
    if T > 1:
        x["length"][1] = T - 1
        x["new_starts"][1, T - 1] = True             # reset exactly at `length`
    ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"],
                                compat=compat)
    new_s, y = run(x, torch.float32, torch.float32, compat)
    assert_close("y", y, ref_y)
    assert_close("new_s", new_s, ref_s)


@pytest.mark.parametrize("T", [1, 4, 8])
@pytest.mark.parametrize("st", [torch.float32, torch.bfloat16])
def test_bf16_io(T, st):
    x = wkv6_inputs(4, T, 3, 64, seed=200 + T, bf16=True, p_reset=0.2)
    if st == torch.bfloat16:
        x["s"] = bf16_round(x["s"]).astype(np.float64)
    ref_s, ref_y = o6.wkv6_base(x["r"], x["k"], x["v"], x["w"], x["u"], x["s"], x["length"], x["new_starts"], compat=True)
    new_s, y = run(x, torch.bfloat16, st, True)
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=1e-5)
    if st == torch.float32:
        assert_close("new_s", new_s, ref_s)
    else:
        assert_close("new_s", new_s, ref_s, rtol=2.0 ** -7, atol=1e-5)


def test_state_layout_is_key_by_value():
    """A one-hot state element S[i][j] must reach y[j] scaled by r[i] and decay by exp(w[i]): a transposed read or
    write of the state fails this."""
    B, T, H, N = 1, 1, 1, 64
    x = wkv6_inputs(B, T, H, N, seed=7, resets=False, lengths=False)
    for n in ("k", "v"):
        x[n][:] = 0.0
    i, j = 5, 41
    x["s"][:] = 0.0
    x["s"][0, 0, i, j] = 2.0
    new_s, y = run(x, torch.float32, torch.float32, False)
    want_y = np.zeros((B, T, H, N))
    want_y[0, 0, 0, j] = 2.0 * x["r"][0, 0, 0, i]
    want_s = np.zeros((B, H, N, N))
    want_s[0, 0, i, j] = 2.0 * np.exp(x["w"][0, 0, 0, i])
    assert_close("y", y, want_y)
    assert_close("new_s", new_s, want_s)


def test_matches_general_kernels():
    x = wkv6_inputs(3, 8, 2, 64, seed=11, p_reset=0.2)
    s_small, y_small = run(x, torch.float32, torch.float32, True)
    s_seq, y_seq = run(x, torch.float32, torch.float32, True, small_t=False)
    assert_close("y", y_small, y_seq)
    assert_close("new_s", s_small, s_seq)


def test_decode_steps_equal_one_prefill_call():
    """Feeding T tokens one at a time with the carried state equals one call over the T tokens."""
    from jaxrwkv_amd import ops
    x = wkv6_inputs(2, 24, 2, 64, seed=300, p_reset=0.1, lengths=False)
    t = {n: dev(x[n]) for n in ("r", "k", "v", "w", "u")}
    ns = dev(x["new_starts"])
    s_full, y_full = ops.wkv6_fwd(t["r"], t["k"], t["v"], t["w"], t["u"], dev(x["s"]), None, ns, compat=False)
    s = dev(x["s"])
    ys = []
    for i in range(24):
        sl = slice(i, i + 1)
        s, y = ops.wkv6_fwd(t["r"][:, sl], t["k"][:, sl], t["v"][:, sl], t["w"][:, sl], t["u"], s, None, ns[:, sl],
                            compat=False)
        ys.append(y)
    torch.cuda.synchronize()
    assert_close("y", host(torch.cat(ys, 1)), host(y_full))
    assert_close("state", host(s), host(s_full))


@pytest.mark.parametrize("io,st", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                   (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("T", [1, 3])
def test_step_on_a_packed_model_state_equals_the_dense_call(io, st, T):
    """hiprwkv_wkv6_step reads and writes a layer's rows of a (B, L, 2+N, C) model state in place (rwkv6.py:148-153,
    221-224): same bits as the dense call on copies of those rows, nothing else of the new model state touched, and an
    update in place (new_s = s) gives the same again."""
    from jaxrwkv_amd import ops
    B, H, N, L, layer = 3, 2, 64, 3, 1
    C = H * N
    x = wkv6_inputs(B, T, H, N, seed=500 + T, bf16=(io == torch.bfloat16), p_reset=0.3)
    x["length"][0] = 0
    t = {n: dev(x[n], io) for n in ("r", "k", "v", "w", "u")}
    length, ns = dev(x["length"]), dev(x["new_starts"])
    g = torch.Generator(device="cuda").manual_seed(7)
    state = (0.1 * torch.randn((B, L, 2 + N, C), device="cuda", generator=g)).to(st)
    new_state = torch.full_like(state, 7.0)
    dense = state[:, layer, 2:].reshape(B, H, N, N).contiguous()
    ref_s, ref_y = ops.wkv6_fwd(t["r"], t["k"], t["v"], t["w"], t["u"], dense, length, ns)
    y = ops.wkv6_step(t["r"], t["k"], t["v"], t["w"], t["u"], state[:, layer, 2:], new_state[:, layer, 2:], length, ns)
    torch.cuda.synchronize()
    assert torch.equal(y, ref_y)
    assert torch.equal(new_state[:, layer, 2:].reshape(B, H, N, N), ref_s)
    untouched = torch.ones_like(new_state, dtype=torch.bool)
    untouched[:, layer, 2:] = False
    assert bool((new_state[untouched] == 7.0).all())
    work = state.clone()
    y2 = ops.wkv6_step(t["r"], t["k"], t["v"], t["w"], t["u"], work[:, layer, 2:], work[:, layer, 2:], length, ns)
    torch.cuda.synchronize()
    assert torch.equal(y2, ref_y)
    assert torch.equal(work[:, layer, 2:].reshape(B, H, N, N), ref_s)
    assert torch.equal(work[untouched], state[untouched])
