"""The small-T (decode) WKV7 kernel, T = 1..8, against the float64 oracle: fp32 arithmetic, so the fp32 bar
(rtol 1e-4 / atol 1e-5) applies to fp32 I/O; with bf16 I/O y is within one bf16 ulp and a bf16 state within one ulp."""
import numpy as np
import pytest
import torch

from oracle import wkv7 as o7
from tests.gpu_util import assert_close, dev, host
from tests.inputs import bf16_round, wkv7_inputs

pytestmark = pytest.mark.gpu


def run(x, io, st, compat):
    from jaxrwkv_amd import ops
    t = {n: dev(x[n], io) for n in ("r", "w", "k", "v", "a", "b")}
    new_s, y, sa = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"], st), dev(x["length"]),
                                dev(x["new_starts"]), compat=compat, want_sa=True)
    torch.cuda.synchronize()
    return host(new_s), host(y), host(sa)


@pytest.mark.parametrize("T", [1, 2, 3, 5, 8])
@pytest.mark.parametrize("compat", [True, False])
def test_fp32(T, compat):
    x = wkv7_inputs(3, T, 2, 64, seed=100 + T, p_reset=0.3, min_len_frac=0.0)
    x["length"][0] = 0
    if T > 1:
        x["length"][1] = T - 1
        x["new_starts"][1, T - 1] = True             # reset exactly at `length`
    ref_s, ref_y, ref_sa = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"],
                                        x["new_starts"], compat=compat, return_sa=True)
    new_s, y, sa = run(x, torch.float32, torch.float32, compat)
    assert_close("y", y, ref_y)
    assert_close("sa", sa, ref_sa)
    assert_close("new_s", new_s, ref_s)


@pytest.mark.parametrize("T", [1, 4, 8])
@pytest.mark.parametrize("st", [torch.float32, torch.bfloat16])
def test_bf16_io(T, st):
    x = wkv7_inputs(4, T, 3, 64, seed=200 + T, bf16=True, p_reset=0.2)
    if st == torch.bfloat16:
        x["s"] = bf16_round(x["s"]).astype(np.float64)
    ref_s, ref_y = o7.wkv7_base(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"], compat=True)
    new_s, y, _ = run(x, torch.bfloat16, st, True)
    assert_close("y", y, ref_y, rtol=2.0 ** -7, atol=1e-5)
    if st == torch.float32:
        assert_close("new_s", new_s, ref_s)
    else:
        assert_close("new_s", new_s, ref_s, rtol=2.0 ** -7, atol=1e-5)


def test_decode_steps_equal_one_prefill_call():
    """Feeding T tokens one at a time with the carried state equals one call over the T tokens."""
    from jaxrwkv_amd import ops
    x = wkv7_inputs(2, 24, 2, 64, seed=300, p_reset=0.1, lengths=False)
    t = {n: dev(x[n]) for n in ("r", "w", "k", "v", "a", "b")}
    ns = dev(x["new_starts"])
    s_full, y_full, _ = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dev(x["s"]), None, ns, compat=False)
    s = dev(x["s"])
    ys = []
    for i in range(24):
        sl = slice(i, i + 1)
        s, y, _ = ops.wkv7_fwd(t["r"][:, sl], t["w"][:, sl], t["k"][:, sl], t["v"][:, sl], t["a"][:, sl], t["b"][:, sl],
                               s, None, ns[:, sl], compat=False)
        ys.append(y)
    torch.cuda.synchronize()
    assert_close("y", host(torch.cat(ys, 1)), host(y_full))
    assert_close("state", host(s), host(s_full))


@pytest.mark.parametrize("io,st", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                   (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("T", [1, 3])
def test_step_on_a_packed_model_state_equals_the_dense_call(io, st, T):
    """hiprwkv_wkv7_step reads and writes a layer's rows of a (B, L, 2+N, C) model state in place (rwkv7.py:176-180,
    254-260): same bits as the dense call on copies of those rows, nothing else of the new model state touched, and
    updating the state in place (new_s = s) gives the same again."""
    from jaxrwkv_amd import ops
    B, H, N, L, layer = 3, 2, 64, 3, 1
    C = H * N
    x = wkv7_inputs(B, T, H, N, seed=400 + T, bf16=(io == torch.bfloat16), p_reset=0.3, min_len_frac=0.0)
    x["length"][0] = 0
    t = {n: dev(x[n], io) for n in ("r", "w", "k", "v", "a", "b")}
    length, ns = dev(x["length"]), dev(x["new_starts"])
    g = torch.Generator(device="cuda").manual_seed(7)
    state = (0.1 * torch.randn((B, L, 2 + N, C), device="cuda", generator=g)).to(st)
    new_state = torch.full_like(state, 7.0)
    dense = state[:, layer, 2:].reshape(B, H, N, N).contiguous()
    ref_s, ref_y, _ = ops.wkv7_fwd(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], dense, length, ns)
    y = ops.wkv7_step(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], state[:, layer, 2:], new_state[:, layer, 2:], length, ns)
    torch.cuda.synchronize()
    assert torch.equal(y, ref_y)
    assert torch.equal(new_state[:, layer, 2:].reshape(B, H, N, N), ref_s)
    untouched = torch.ones_like(new_state, dtype=torch.bool)
    untouched[:, layer, 2:] = False
    assert bool((new_state[untouched] == 7.0).all())
    work = state.clone()
    y2 = ops.wkv7_step(t["r"], t["w"], t["k"], t["v"], t["a"], t["b"], work[:, layer, 2:], work[:, layer, 2:], length, ns)
    torch.cuda.synchronize()
    assert torch.equal(y2, ref_y)
    assert torch.equal(work[:, layer, 2:].reshape(B, H, N, N), ref_s)
    untouched[:, layer, 2:] = False
    assert torch.equal(work[untouched], state[untouched])
