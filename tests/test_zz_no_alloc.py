"""hiprwkv_wkv4_bwd_noalloc (the WKV4 backward with its checkpoint workspace inside the library's device image)
against hiprwkv_wkv4_bwd with a caller-allocated workspace, through the C ABI: bit-identical cotangents on two calls
in a row, the second on a smaller input (the scratch array then still holds the first call's checkpoints), and the
size limit is refused with HIPRWKV_ENOSPACE."""
import ctypes

import numpy as np
import pytest
import torch

from tests.inputs import wkv4_inputs

pytestmark = pytest.mark.gpu


def both_entry_points(B, T, C, seed):
    from jaxrwkv_amd import _lib
    lib = _lib.load()
    x = wkv4_inputs(B, T, C, seed=seed, p_reset=0.05, default_state=False, min_len=1)
    g = np.random.default_rng(seed)
    f = lambda a: torch.from_numpy(np.ascontiguousarray(a)).float().cuda()
    w, u, k, v, s = (f(x[n]) for n in ("w", "u", "k", "v", "s"))
    gy, gs_new = f(g.standard_normal((B, T, C))), f(g.standard_normal((B, 3, C)))
    length = torch.from_numpy(x["length"]).cuda().to(torch.int32)
    ns = torch.from_numpy(x["new_starts"]).cuda()
    stream = torch.cuda.current_stream().cuda_stream
    p = lambda t: ctypes.c_void_p(t.data_ptr())

    def outputs():
        return (torch.full((B, C), float("nan"), device="cuda"), torch.full((B, C), float("nan"), device="cuda"),
                torch.full_like(k, float("nan")), torch.full_like(v, float("nan")), torch.full_like(s, float("nan")))

    ref = outputs()
    nbytes = lib.hiprwkv_wkv4_bwd_workspace_bytes(B, T, C)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    rc = lib.hiprwkv_wkv4_bwd(stream, _lib.F32, B, T, C, p(w), p(u), p(k), p(v), p(gy), p(s), p(length), p(ns),
                              p(gs_new), *(p(t) for t in ref), p(ws), nbytes, _lib.COMPAT_ASSOC)
    _lib.check(rc, "hiprwkv_wkv4_bwd")
    got = outputs()
    rc = lib.hiprwkv_wkv4_bwd_noalloc(stream, _lib.F32, B, T, C, p(w), p(u), p(k), p(v), p(gy), p(s), p(length),
                                      p(ns), p(gs_new), *(p(t) for t in got), _lib.COMPAT_ASSOC)
    _lib.check(rc, "hiprwkv_wkv4_bwd_noalloc")
    torch.cuda.synchronize()
    return ref, got


def test_noalloc_entry_point_equals_the_workspace_one_on_two_calls_in_a_row():
    for B, T, C, seed in ((3, 130, 100, 61), (2, 40, 64, 62)):     # the second call is the smaller one
        ref, got = both_entry_points(B, T, C, seed)
        for name, r, g in zip(("gw", "gu", "gk", "gv", "gs"), ref, got):
            assert torch.isfinite(r).all(), name
            assert torch.equal(r, g), name


def test_noalloc_entry_point_refuses_shapes_beyond_its_scratch():
    from jaxrwkv_amd import _lib
    lib = _lib.load()
    limit = lib.hiprwkv_wkv4_bwd_noalloc_max_bytes()
    assert limit == 16 << 20
    B, T, C = 32, 4096, 2560
    assert lib.hiprwkv_wkv4_bwd_workspace_bytes(B, T, C) > limit
    ok = ctypes.c_void_p(0x10000)
    rc = lib.hiprwkv_wkv4_bwd_noalloc(None, _lib.F32, B, T, C, *([ok] * 6), None, None, None, *([ok] * 5), 0)
    assert rc == -3 and b"scratch" in lib.hiprwkv_last_error()
