"""The RWKV-7 full-model harness (torch plumbing + HipRWKV.inner_loop) against the float64 full-model oracle on the
same weights: logits and final state.  fp32 models use the sequential fp32 kernels, bf16 models the chunked ones.

Weights come from the harness's own seeded initialisation (the reference's threefry streams cannot be reproduced
without jax), with the zero-initialised matrices replaced by small random ones so that the recurrence reaches the
logits.  Tolerances: fp32 -- logits and state within 1e-3 of their rms (fp32 GEMMs of 2 to 12 layers against
float64); bf16 -- total-variation distance of the softmax of the logits below 2e-2 per token and state within
3e-2 of its rms (every activation is rounded to bf16 in the harness, which dominates; the op-level bf16 bar is
checked in tests/test_gpu_wkv7_chunked.py).
"""
import numpy as np
import pytest
import torch

from oracle import model7 as om
from tests.gpu_util import host

pytestmark = pytest.mark.gpu


def softmax(z):
    z = z - z.max(-1, keepdims=True)
    e = np.exp(z)
    return e / e.sum(-1, keepdims=True)


def run_case(L, C, vocab, B, T, dtype, seed, p_reset=0.05, state_scale=0.0):
    from jaxrwkv_amd.model7 import RWKV7, randomize_weights, tree_map
    params = randomize_weights(seed, L, C, vocab, dtype=dtype, device="cuda", zero_init=False)
    g = np.random.default_rng(seed)
    tokens = g.integers(0, vocab, size=(B, T))
    ns = g.random((B, T)) < p_reset
    length = g.integers(max(1, T // 2), T + 1, size=(B,))
    state = RWKV7.default_state(params, B)
    if state_scale:
        state = (state_scale * torch.randn(state.shape, device="cuda", generator=torch.Generator("cuda").manual_seed(seed))).to(dtype)
    logits, new_state = RWKV7.forward(params, torch.from_numpy(tokens).cuda(), state,
                                      torch.from_numpy(length).cuda(), torch.from_numpy(ns).cuda())
    torch.cuda.synchronize()
    p64 = om.to_f64(tree_map(lambda t: t.float().cpu().numpy(), params))
    st64 = host(state)
    ref_logits, ref_state = [], []
    for b in range(B):
        lg, st = om.forward(p64, tokens[b], st64[b], int(length[b]), ns[b])
        ref_logits.append(lg)
        ref_state.append(st)
    return host(logits), host(new_state), np.stack(ref_logits), np.stack(ref_state)


def rel_rms(a, b):
    return float(np.sqrt(np.mean((a - b) ** 2)) / max(np.sqrt(np.mean(b ** 2)), 1e-30))


def test_small_fp32_model_with_resets_lengths_and_carried_state():
    lg, st, rlg, rst = run_case(L=3, C=128, vocab=211, B=3, T=45, dtype=torch.float32, seed=5, state_scale=0.1)
    assert rel_rms(lg, rlg) < 1e-3 and np.abs(lg - rlg).max() < 1e-3 * np.sqrt(np.mean(rlg ** 2)) * 10
    assert rel_rms(st, rst) < 1e-3


def test_small_bf16_model():
    lg, st, rlg, rst = run_case(L=2, C=128, vocab=211, B=2, T=70, dtype=torch.bfloat16, seed=6)
    tvd = 0.5 * np.abs(softmax(lg) - softmax(rlg)).sum(-1)
    assert tvd.max() < 2e-2, tvd.max()
    assert rel_rms(st, rst) < 3e-2


def test_rwkv7_0p1b_shape_fp32():
    """BASELINE configs[0]: L=12, C=768, H=12, head size 64, vocab 65536, fp32, B=1, T=512, default zero state."""
    lg, st, rlg, rst = run_case(L=12, C=768, vocab=65536, B=1, T=512, dtype=torch.float32, seed=7, p_reset=0.0)
    assert rel_rms(lg, rlg) < 1e-3, rel_rms(lg, rlg)
    assert rel_rms(st, rst) < 1e-3, rel_rms(st, rst)
    tvd = 0.5 * np.abs(softmax(lg) - softmax(rlg)).sum(-1)
    assert tvd.max() < 1e-3, tvd.max()


def test_decode_step_in_a_hip_graph_replays_like_eager():
    """A captured decode step (B=8, T=1) replayed several times with new tokens and the carried state, with eager work
    and synchronisations between the replays, equals the eager step every time."""
    from jaxrwkv_amd.model7 import RWKV7, randomize_weights
    params = randomize_weights(11, 2, 128, 211, dtype=torch.bfloat16, device="cuda", zero_init=False)
    B = 8
    gen = torch.Generator("cuda").manual_seed(3)
    tok = torch.randint(0, 211, (B, 1), device="cuda", generator=gen)
    state = (0.1 * torch.randn((B, 2, 66, 128), device="cuda", generator=gen)).bfloat16()

    def step():
        with torch.no_grad():
            return RWKV7.forward(params, tok, state, None, None)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        g_logits, g_state = step()
    for it in range(4):
        tok.copy_(torch.randint(0, 211, (B, 1), device="cuda", generator=gen))
        e_logits, e_state = step()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(g_logits, e_logits), it
        assert torch.equal(g_state, e_state), it
        state.copy_(e_state)                          # carry the state into the next step
