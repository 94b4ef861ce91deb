"""Helpers of the GPU parity tests: upload seeded inputs, call the C ABI via jaxrwkv_amd.ops, compare to the oracle."""
import numpy as np
import torch

FP32_RTOL, FP32_ATOL = 1e-4, 1e-5      # the stated fp32 bar for y and the final state


def dev(x, dtype=torch.float32):
    if x.dtype == bool:
        return torch.from_numpy(np.ascontiguousarray(x)).cuda()
    if np.issubdtype(x.dtype, np.integer):
        return torch.from_numpy(np.ascontiguousarray(x)).cuda()
    return torch.from_numpy(np.ascontiguousarray(x)).to(dtype).cuda()


def host(t):
    return t.detach().float().cpu().numpy().astype(np.float64)


def assert_close(name, got, ref, rtol=FP32_RTOL, atol=FP32_ATOL, scale_atol=False):
    got, ref = np.asarray(got, np.float64), np.asarray(ref, np.float64)
    a = atol * (max(1.0, float(np.sqrt(np.mean(ref ** 2)))) if scale_atol else 1.0)
    err = np.abs(got - ref)
    bad = err > a + rtol * np.abs(ref)
    if bad.any():
        i = np.unravel_index(np.argmax(err - (a + rtol * np.abs(ref))), err.shape)
        raise AssertionError(f"{name}: {bad.sum()} of {bad.size} elements out of tolerance; worst at {i}: "
                             f"got {got[i]!r}, want {ref[i]!r} (rtol {rtol}, atol {a})")


def tvd_of_projected(y_a, y_b, vocab=512, seed=0):
    """Total-variation distance of softmax(groupnorm(y) @ P) for a fixed random projection P: the op-level proxy
    of 'logits TVD' (the model applies a per-head group norm to y, rwkv7.py:263, before any projection)."""
    g = np.random.default_rng(seed)
    C = y_a.shape[-2] * y_a.shape[-1]
    P = g.standard_normal((C, vocab)) / np.sqrt(C)
    def sm(y):
        y = (y - y.mean(-1, keepdims=True)) / np.sqrt(y.var(-1, keepdims=True) + 64e-5)
        z = y.reshape(y.shape[0], y.shape[1], C) @ P
        z = z - z.max(-1, keepdims=True)
        e = np.exp(z)
        return e / e.sum(-1, keepdims=True)
    return 0.5 * np.abs(sm(y_a) - sm(y_b)).sum(-1)
