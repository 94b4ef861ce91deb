"""Benchmark of the WKV7 hot path on one MI355X:  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward pass of the isolated WKV7 op over one synthetic batch of the headline shape
(B=8, T=4096, H=32, N=64, bf16 I/O, fp32 state, new_starts ~ Bernoulli(1/1024), length ~ U{T/2..T}); inputs are
resident in HBM before the timed region.  Prints ONE JSON line: forward tokens/s as `value`, forward+backward
tokens/s beside it, the HBM roofline of the dominant kernel and a bounded CPU baseline (the oracle's
associative-scan restatement on the host cores).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import numpy as np  # noqa: E402

HBM_PEAK_GBS = 8000.0
B, T, H, N = 8, 4096, 32, 64


def make_inputs(torch, seed=0):
    """Config-2 inputs, generated on the host with a fixed stream and uploaded once."""
    g = np.random.default_rng(seed)
    shp = (B, T, H, N)
    f = lambda x: torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).cuda()
    r = f(g.standard_normal(shp, dtype=np.float32)).bfloat16()
    k = f(g.standard_normal(shp, dtype=np.float32)).bfloat16()
    v = f(g.standard_normal(shp, dtype=np.float32)).bfloat16()
    w = f(-0.5 + 0.5 * g.standard_normal(shp, dtype=np.float32)).bfloat16()
    kap = g.standard_normal(shp, dtype=np.float32)
    kap /= np.linalg.norm(kap, axis=-1, keepdims=True)
    a = f(-kap).bfloat16()
    b = f(kap / (1.0 + np.exp(-g.standard_normal(shp, dtype=np.float32)))).bfloat16()
    s = f(0.1 * g.standard_normal((B, H, N, N), dtype=np.float32))
    ns = torch.from_numpy(g.random((B, T)) < 1.0 / 1024).cuda()
    length = torch.from_numpy(g.integers(T // 2, T + 1, size=(B,)).astype(np.int32)).cuda()
    dy = f(g.standard_normal(shp, dtype=np.float32)).bfloat16()
    return dict(r=r, w=w, k=k, v=v, a=a, b=b, s=s, new_starts=ns, length=length, dy=dy)


def time_region(torch, fn, steps, warmup):
    """Wall time of exactly `steps` calls, bracketed by device syncs, plus per-call HIP-event durations."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
    t0 = time.perf_counter()
    for e0, e1 in evs:
        e0.record()
        fn()
        e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    per_call_ms = [e0.elapsed_time(e1) for e0, e1 in evs]
    return wall, per_call_ms


def cpu_baseline(sample_heads=2, threads=None):
    """Oracle's AssociativeScanRWKV restatement (log-depth scan, fp32) on the host: one sequence of the benchmark
    shape restricted to `sample_heads` of the 32 heads; tokens/s is scaled to all heads of a token."""
    from oracle import wkv7 as o7
    g = np.random.default_rng(1)
    shp = (1, T, sample_heads, N)
    r, k, v = (g.standard_normal(shp) for _ in range(3))
    w = -0.5 + 0.5 * g.standard_normal(shp)
    kap = g.standard_normal(shp)
    kap /= np.linalg.norm(kap, axis=-1, keepdims=True)
    a, b = -kap, kap / (1.0 + np.exp(-g.standard_normal(shp)))
    s = 0.1 * g.standard_normal((1, sample_heads, N, N))
    ns = g.random((1, T)) < 1.0 / 1024
    t0 = time.perf_counter()
    o7.wkv7_assoc_scan(r, w, k, v, a, b, s, np.array([T]), ns, dtype=np.float32)
    dt = time.perf_counter() - t0
    tok_s = T * (sample_heads / H) / dt
    return {"value": tok_s, "unit": "tokens/s", "cores": threads or (os.cpu_count() or 1), "kind": "port",
            "sample": f"1 sequence, T={T}, {sample_heads} of {H} heads, fp32 log-depth associative scan "
                      f"(oracle.wkv7.wkv7_assoc_scan, NumPy/BLAS threads), {dt:.1f} s, scaled by heads"}


def cpu_baseline_sequential(tokens=1024):
    """Second CPU number: the oracle's sequential O(T N^2) recurrence (float64 NumPy), all 32 heads of one sequence."""
    from oracle import wkv7 as o7
    g = np.random.default_rng(2)
    shp = (1, tokens, H, N)
    r, k, v = (g.standard_normal(shp) for _ in range(3))
    w = -0.5 + 0.5 * g.standard_normal(shp)
    kap = g.standard_normal(shp)
    kap /= np.linalg.norm(kap, axis=-1, keepdims=True)
    a, b = -kap, kap / (1.0 + np.exp(-g.standard_normal(shp)))
    s = 0.1 * g.standard_normal((1, H, N, N))
    t0 = time.perf_counter()
    o7.wkv7_base(r, w, k, v, a, b, s)
    dt = time.perf_counter() - t0
    return {"value": tokens / dt, "unit": "tokens/s", "cores": 1, "kind": "port",
            "sample": f"1 sequence, T={tokens}, all {H} heads, float64 sequential loop (oracle.wkv7.wkv7_base), {dt:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-bwd", action="store_true")
    ap.add_argument("--seq", action="store_true", help="force the sequential fp32 VALU kernel")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three 1 GiB device copies before the timed region (scale for rocprofv3 --pmc)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (the op shards over batch/heads "
              "without communication); run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    from jaxrwkv_amd import _lib, ops
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    _lib.load()
    x = make_inputs(torch)
    tokens = B * T

    if args.copy_probe:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    def fwd():
        return ops.wkv7_fwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"],
                            compat=True, want_sa=False, force_seq=args.seq)

    wall, per_call = time_region(torch, fwd, args.steps, args.warmup)
    ms_step = 1e3 * wall / args.steps
    kern_ms = float(np.mean(per_call))
    fwd_bytes = 7 * tokens * H * N * 2 + 2 * B * H * N * N * 4 + B * T + B * 4
    achieved = fwd_bytes / (kern_ms * 1e-3) / 1e9

    out = {
        "metric": "WKV7 fwd tokens/s (B8 T4096 H32 N64 bf16)", "value": tokens / (ms_step * 1e-3), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16 I/O, fp32 state/accumulate",
        "data": "synthetic",
        "config": {"workload": "isolated WKV7 op, B=8 T=4096 H=32 N=64, bf16 r/w/k/v/a/b, fp32 state, "
                               "new_starts~Bernoulli(1/1024), length~U{T/2..T} (BASELINE configs[1])",
                   "kernel": "sequential" if args.seq else "default"},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": None,
                     "kernel_ms": kern_ms, "algorithmic_bytes": fwd_bytes},
    }

    if not args.no_bwd:
        def fwd_bwd():
            new_s, y, sa = ops.wkv7_fwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"],
                                        x["new_starts"], compat=True, want_sa=True)
            return ops.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"],
                                x["dy"], sa, None, compat=True)
        wall2, _ = time_region(torch, fwd_bwd, max(2, args.steps // 4), 1)
        ms2 = 1e3 * wall2 / max(2, args.steps // 4)
        fb_bytes = 20 * tokens * H * N * 2 + 4 * B * H * N * N * 4
        out["fwd_bwd"] = {"tokens_per_s": tokens / (ms2 * 1e-3), "ms_per_step": ms2,
                          "hbm_frac": fb_bytes / (ms2 * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": fb_bytes}
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        out["cpu_baseline_sequential"] = cpu_baseline_sequential()
        out["gpu_over_cpu"] = out["value"] / out["cpu_baseline"]["value"]
    print(json.dumps(out))


if __name__ == "__main__":
    main()
