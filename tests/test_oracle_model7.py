"""Pins the full-model oracle (oracle/model7.py) by properties the architecture fixes, on a small random model."""
import numpy as np
import pytest
import torch

from oracle import model7 as om


def small_model(seed=0, L=2, C=128, vocab=97, zero_init=False):
    from jaxrwkv_amd.model7 import randomize_weights, tree_map
    p = randomize_weights(seed, L, C, vocab, dtype=torch.float32, device="cpu", zero_init=zero_init)
    return tree_map(lambda t: t.numpy().astype(np.float64), p)


@pytest.fixture(scope="module")
def model():
    return small_model()


def toks(T, vocab=97, seed=1):
    return np.random.default_rng(seed).integers(0, vocab, size=T)


def test_norm_layers_match_torch_definitions():
    g = np.random.default_rng(0)
    x = g.standard_normal((5, 128))
    w = {"weight": g.standard_normal(128), "bias": g.standard_normal(128)}
    ref = torch.nn.functional.layer_norm(torch.from_numpy(x), (128,), torch.from_numpy(w["weight"]),
                                         torch.from_numpy(w["bias"]), 1e-5).numpy()
    np.testing.assert_allclose(om.layer_norm(x, w), ref, rtol=1e-10, atol=1e-12)
    ref = torch.nn.functional.group_norm(torch.from_numpy(x), 2, torch.from_numpy(w["weight"]),
                                         torch.from_numpy(w["bias"]), 64e-5).numpy()
    np.testing.assert_allclose(om.group_norm_tokens(x, 2, w["weight"], w["bias"], 64e-5), ref, rtol=1e-10, atol=1e-12)


def test_split_sequence_with_carried_state(model):
    t = toks(23)
    s0 = om.default_state(model)
    full, s_full = om.forward(model, t, s0)
    a, s_a = om.forward(model, t[:9], s0)
    b, s_b = om.forward(model, t[9:], s_a)
    np.testing.assert_allclose(np.concatenate([a, b]), full, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(s_b, s_full, rtol=1e-9, atol=1e-10)


def test_reset_equals_fresh_run(model):
    t = toks(20)
    ns = np.zeros(20, bool)
    ns[12] = True
    s0 = om.default_state(model)
    s_junk = np.random.default_rng(3).standard_normal(s0.shape)
    out, s_out = om.forward(model, t, s_junk, new_starts=ns)
    fresh, s_fresh = om.forward(model, t[12:], s0)
    np.testing.assert_allclose(out[12:], fresh, rtol=1e-9, atol=1e-10)
    np.testing.assert_allclose(s_out, s_fresh, rtol=1e-9, atol=1e-10)


def test_length_equals_truncated_run(model):
    t = toks(18)
    s0 = om.default_state(model)
    _, s_len = om.forward(model, t, s0, length=11)
    _, s_trunc = om.forward(model, t[:11], s0)
    np.testing.assert_allclose(s_len, s_trunc, rtol=1e-9, atol=1e-10)


def test_reference_initialisation_makes_blocks_vanish():
    m = small_model(zero_init=True)
    t = toks(7)
    logits, state = om.forward(m, t, om.default_state(m))
    x = om.layer_norm(m["emb"]["weight"][t], m["ln0"])
    np.testing.assert_allclose(logits, om.layer_norm(x, m["ln_out"]) @ m["head"]["weight"].T, rtol=1e-12, atol=1e-12)
    assert np.abs(state[:, 2:]).max() > 0          # the recurrence still ran


# ---- special cases that pin the formulas of time_mixing_seq / channel_mixing_seq (rwkv7.py:190-198, 223-267): a
#      wrong sign in the decay, exchanged k_k / k_a, a wrong v_first mix or bonus term fails one of them.  The
#      operands the block hands to the recurrence are observed through a stand-in for oracle.wkv7.wkv7_base, and
#      the expected values are formed independently with torch.nn.functional in float64.
class Spy:
    def __init__(self, monkeypatch, zero_out=False):
        self.calls = []
        real = om.o7.wkv7_base

        def fake(r, w, k, v, a, b, s, length, new_starts, compat=True):
            self.calls.append(dict(r=r[0], w=w[0], k=k[0], v=v[0], a=a[0], b=b[0]))
            s_new, out = real(r, w, k, v, a, b, s, length, new_starts, compat=compat)
            return s_new, (np.zeros_like(out) if zero_out else out)
        monkeypatch.setattr(om.o7, "wkv7_base", fake)


def att_of(model, layer):
    return om._layer(model["blocks"], layer)["att"]


def time_mix(model, layer, x, v_first, T, att=None):
    att = att or att_of(model, layer)
    L, H, S = model["blocks"]["att"]["r_k"].shape
    state = np.zeros((1 + S, x.shape[1]))
    return om.time_mixing_seq(x, state, v_first, att, T, np.zeros(T, bool), H, S, layer)


def tt(x):
    return torch.from_numpy(np.ascontiguousarray(x))


def test_decay_argument_is_bounded_and_reduces_to_w0(model, monkeypatch):
    spy = Spy(monkeypatch)
    T, C = 9, 128
    x = np.random.default_rng(5).standard_normal((T, C))
    time_mix(model, 1, x, x, T)
    w = spy.calls[-1]["w"].reshape(T, C)
    assert np.all(w <= -0.5)                                   # rwkv7.py:236: -softplus(.) - 0.5
    att = dict(att_of(model, 1))
    att["w1"] = np.zeros_like(att["w1"])
    time_mix(model, 1, x, x, T, att)
    expect = -0.5 - torch.nn.functional.softplus(-tt(att["w0"])).numpy()
    np.testing.assert_allclose(spy.calls[-1]["w"].reshape(T, C), np.broadcast_to(expect, (T, C)), rtol=1e-12)


def test_key_scaling_removal_vector_and_its_gate(model, monkeypatch):
    spy = Spy(monkeypatch)
    T, C = 7, 128
    x = np.random.default_rng(6).standard_normal((T, C))
    att = dict(att_of(model, 0))
    att["x_k"] = np.zeros_like(att["x_k"])                     # no token shift in the key path: xk = x
    k_plain = (tt(x) @ tt(att["key"]["weight"]).T).numpy()
    # a == 1 (a0 -> +inf, no LoRA): k' = k ; the removal vector is -normalize(k k_k) per head, b = kk a = kk
    a1 = dict(att)
    a1["a0"] = np.full_like(att["a0"], 50.0)
    a1["a1"] = np.zeros_like(att["a1"])
    time_mix(model, 0, x, x, T, a1)
    c = spy.calls[-1]
    np.testing.assert_allclose(c["k"].reshape(T, C), k_plain, rtol=1e-10, atol=1e-12)
    kk = torch.nn.functional.normalize((tt(k_plain) * tt(att["k_k"])).reshape(T, 2, 64), dim=-1).numpy()
    np.testing.assert_allclose(c["a"], -kk, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(c["b"], kk, rtol=1e-10, atol=1e-12)
    # k_a == 0: k' = k whatever a is; b = kk sigmoid(a0 + ...)
    a2 = dict(att)
    a2["k_a"] = np.zeros_like(att["k_a"])
    a2["a1"] = np.zeros_like(att["a1"])
    time_mix(model, 0, x, x, T, a2)
    c = spy.calls[-1]
    np.testing.assert_allclose(c["k"].reshape(T, C), k_plain, rtol=1e-10, atol=1e-12)
    gate = torch.sigmoid(tt(att["a0"])).numpy().reshape(2, 64)
    np.testing.assert_allclose(c["b"], kk * gate, rtol=1e-10, atol=1e-12)
    # general a, k_a: k' = k (1 + (a - 1) k_a)
    a3 = dict(att)
    a3["a1"] = np.zeros_like(att["a1"])
    time_mix(model, 0, x, x, T, a3)
    expect = k_plain * (1 + (torch.sigmoid(tt(att["a0"])).numpy() - 1) * att["k_a"])
    np.testing.assert_allclose(spy.calls[-1]["k"].reshape(T, C), expect, rtol=1e-10, atol=1e-12)


def test_value_residual_mix(model, monkeypatch):
    spy = Spy(monkeypatch)
    T, C = 6, 128
    g = np.random.default_rng(7)
    x, vf = g.standard_normal((T, C)), g.standard_normal((T, C))
    att0 = dict(att_of(model, 0))
    att0["x_v"] = np.zeros_like(att0["x_v"])
    v_plain = (tt(x) @ tt(att0["value"]["weight"]).T).numpy()
    _, _, v_first = time_mix(model, 0, x, vf, T, att0)        # layer 0: v_first is this layer's v
    np.testing.assert_allclose(v_first, v_plain, rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(spy.calls[-1]["v"].reshape(T, C), v_plain, rtol=1e-10, atol=1e-12)
    att1 = dict(att_of(model, 1))
    att1["v1"] = np.zeros_like(att1["v1"])
    att1["v0"] = np.full_like(att1["v0"], 50.0)                # gate -> 1: v = v_first
    _, _, v_out = time_mix(model, 1, x, vf, T, att1)
    np.testing.assert_allclose(spy.calls[-1]["v"].reshape(T, C), vf, rtol=1e-10, atol=1e-10)
    np.testing.assert_allclose(v_out, vf)                      # passed on unchanged
    att1["v0"] = np.full_like(att1["v0"], -50.0)               # gate -> 0: v = this layer's own projection
    att1["x_v"] = np.zeros_like(att1["x_v"])
    time_mix(model, 1, x, vf, T, att1)
    own = (tt(x) @ tt(att1["value"]["weight"]).T).numpy()
    np.testing.assert_allclose(spy.calls[-1]["v"].reshape(T, C), own, rtol=1e-10, atol=1e-10)


def test_gate_bonus_and_output_projection(model, monkeypatch):
    T, C = 5, 128
    x = np.random.default_rng(8).standard_normal((T, C))
    att = dict(att_of(model, 1))
    g0 = dict(att)
    g0["g2"] = np.zeros_like(att["g2"])                        # gate == 0: the block contributes nothing
    out, _, _ = time_mix(model, 1, x, x, T, g0)
    assert np.all(out == 0.0)
    # recurrence output replaced by zeros: group norm gives its bias; what is left is (bias + bonus) g Wo^T
    spy = Spy(monkeypatch, zero_out=True)
    att["ln_x"] = {"weight": att["ln_x"]["weight"], "bias": np.random.default_rng(9).standard_normal(C)}
    out, _, _ = time_mix(model, 1, x, x, T, att)
    c = spy.calls[-1]
    xg = tt(x + (np.concatenate([np.zeros((1, C)), x[:-1]]) - x) * att["x_g"])
    gate = (torch.sigmoid(xg @ tt(att["g1"])) @ tt(att["g2"])).numpy()
    bonus = ((tt(c["r"]) * tt(c["k"]) * tt(att["r_k"])).sum(-1, keepdim=True) * tt(c["v"])).numpy().reshape(T, C)
    expect = ((att["ln_x"]["bias"] + bonus) * gate) @ att["output"]["weight"].T
    np.testing.assert_allclose(out, expect, rtol=1e-9, atol=1e-12)
    nob = dict(att)
    nob["r_k"] = np.zeros_like(att["r_k"])                     # r_k == 0: no bonus
    out, _, _ = time_mix(model, 1, x, x, T, nob)
    np.testing.assert_allclose(out, (att["ln_x"]["bias"] * gate) @ att["output"]["weight"].T, rtol=1e-9, atol=1e-12)


def test_channel_mix_without_token_shift_is_a_relu_squared_mlp(model):
    T, C = 8, 128
    x = np.random.default_rng(10).standard_normal((T, C))
    ffn = dict(om._layer(model["blocks"], 0)["ffn"])
    ffn["x_k"] = np.zeros_like(ffn["x_k"])
    out, last = om.channel_mixing_seq(x, np.zeros((1, C)), ffn, 5, np.zeros(T, bool))
    F = torch.nn.functional
    ref = F.linear(F.relu(F.linear(tt(x), tt(ffn["key"]["weight"]))) ** 2, tt(ffn["value"]["weight"])).numpy()
    np.testing.assert_allclose(out, ref, rtol=1e-10, atol=1e-12)
    np.testing.assert_array_equal(last, x[4])
    # with the shift: xk = x + (prev - x) x_k, prev = state row for t = 0 and zero at a reset
    ffn = om._layer(model["blocks"], 0)["ffn"]
    ns = np.zeros(T, bool)
    ns[3] = True
    st = np.random.default_rng(11).standard_normal((1, C))
    out, _ = om.channel_mixing_seq(x, st, ffn, T, ns)
    prev = np.concatenate([st, x[:-1]])
    prev[3] = 0.0
    xk = tt(x + (prev - x) * ffn["x_k"])
    ref = F.linear(F.relu(F.linear(xk, tt(ffn["key"]["weight"]))) ** 2, tt(ffn["value"]["weight"])).numpy()
    np.testing.assert_allclose(out, ref, rtol=1e-10, atol=1e-12)


def test_bf16_op_io_rounds_the_six_inputs_and_the_output_and_nothing_else(model, monkeypatch):
    """forward(op_io="bf16"): the recurrence sees bf16-representable r, w, k, v, a, b (the same values as without the
    option, rounded to nearest even), its output is rounded before the group norm, and the bonus term, the state and
    every projection stay float64."""
    from tests.inputs import bf16_round
    spy = Spy(monkeypatch)
    T, C = 11, 128
    x = np.random.default_rng(9).standard_normal((T, C))
    L, H, S = model["blocks"]["att"]["r_k"].shape
    state = 0.1 * np.random.default_rng(10).standard_normal((1 + S, C))
    att = att_of(model, 1)
    exact = om.time_mixing_seq(x, state, x, att, T, np.zeros(T, bool), H, S, 1)
    plain = spy.calls[-1]
    rounded = om.time_mixing_seq(x, state, x, att, T, np.zeros(T, bool), H, S, 1, op_io="bf16")
    seen = spy.calls[-1]
    for n in "rwkvab":
        np.testing.assert_array_equal(seen[n], bf16_round(plain[n]).astype(np.float64))
        assert np.any(seen[n] != plain[n])
    rel = lambda a, b: np.sqrt(np.mean((a - b) ** 2) / np.mean(b ** 2))
    assert 1e-4 < rel(rounded[0], exact[0]) < 2e-2             # bf16 rounding of the op's I/O, nothing coarser
    assert rel(rounded[1][1:], exact[1][1:]) < 2e-2 and np.array_equal(rounded[1][0], exact[1][0])
    # with an output projection that reads the bonus term only (zero group-norm weight and bias), y does not depend on
    # the op's output at all: the option must not touch that path
    att0 = dict(att)
    att0["ln_x"] = {"weight": np.zeros_like(att["ln_x"]["weight"]), "bias": np.zeros_like(att["ln_x"]["bias"])}
    a0 = om.time_mixing_seq(x, state, x, att0, T, np.zeros(T, bool), H, S, 1)
    b0 = om.time_mixing_seq(x, state, x, att0, T, np.zeros(T, bool), H, S, 1, op_io="bf16")
    np.testing.assert_array_equal(a0[0], b0[0])
