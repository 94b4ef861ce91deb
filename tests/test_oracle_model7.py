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
