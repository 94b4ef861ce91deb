"""Benchmark of the WKV hot path on one MI355X:  python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one forward pass of the isolated WKV7 op over one synthetic batch of the headline shape
(B=8, T=4096, H=32, N=64, bf16 I/O, fp32 state, new_starts ~ Bernoulli(1/1024), length ~ U{T/2..T}); inputs are
resident in HBM before the timed region.  Prints ONE JSON line: forward tokens/s as `value`, forward+backward
tokens/s beside it, the HBM roofline of the dominant kernel and a bounded CPU baseline (the oracle's
associative-scan restatement on the host cores).

`--workload wkv6` / `--workload wkv4` time the two secondary ops (B=16 T=2048 H=32 N=64 bf16, and B=32 T=4096
C=2560 fp32) with the same JSON layout; `--workload model7` runs the RWKV-7 1.5B-shaped full model through the torch
harness (prefill B=16 T=4096, decode B=256 single-token steps, eager and from a captured HIP graph).  The default,
and the line the headline metric is quoted on, is wkv7.
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
# HBM bytes per forward launch from `rocprofv3 --pmc FETCH_SIZE` / `WRITE_SIZE` (scaled by a 1 GiB copy; commands and
# figures in profiles/), each with the sha1 prefix of the kernel source it was measured on: when the source has
# changed since, `roofline.traffic` is null instead of a stale figure.
MEASURED_TRAFFIC = {
    "wkv7_fwd": (948.7e6, "wkv7_fwd.hip", "51a3d3ca403c", "profiles/wkv7_fwd_B8_T4096_H32_bf16.md"),
    "wkv4_fwd": (4028.7e6, "wkv4.hip", "d83a0992a92e", "profiles/wkv4_fwd_B32_T4096_C2560_f32.md"),
    "wkv6_fwd": (688.4e6, "wkv6_fwd.hip", "e577f9812ac6", "profiles/wkv6_fwd_bwd_B16_T2048_H32_bf16.md"),
}


def measured_traffic(name):
    """(bytes, source) of the counter run recorded in profiles/: `roofline.traffic` is NOT measured by this run, it
    is the figure of the named profile, given only while the kernel source still has the hash it was measured on."""
    import hashlib
    nbytes, src, sha, profile = MEASURED_TRAFFIC[name]
    path = os.path.join(ROOT, "jaxrwkv_amd", "csrc", src)
    now = hashlib.sha1(open(path, "rb").read()).hexdigest()[:12]
    if sha != now:
        return None, f"{profile} (stale: {src} has changed since the counter run)"
    return nbytes, f"{profile} (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not measured by this run)"


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


PREWARM_S = 0.3


def time_region(torch, fn, steps, warmup, prewarm_s=PREWARM_S):
    """Wall time of exactly `steps` calls, bracketed by device syncs, and the HIP-event time of the same region
    (events recorded on the stream the kernels are launched on) divided by `steps`.

    Before the `warmup` untimed steps the same call is repeated for `prewarm_s` seconds, untimed as well: the GPU
    raises its clocks over the first tens of milliseconds of work (the first 20 launches of the headline kernel
    take 0.41 ms each, launches 100-600 take 0.32 ms), and the figure wanted is the steady one."""
    t_end = time.perf_counter() + prewarm_s
    batch = 1
    while prewarm_s > 0 and time.perf_counter() < t_end:
        t0 = time.perf_counter()
        for _ in range(batch):
            fn()
        torch.cuda.synchronize()
        batch = 8 if time.perf_counter() - t0 < 0.02 else 1
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) / steps


def cpu_baseline(sample_heads=2, threads=None, target_s=15.0, max_heads=32):
    """Oracle's AssociativeScanRWKV restatement (log-depth scan, fp32) on the host: one sequence of the benchmark
    shape restricted to a few of the 32 heads; tokens/s is scaled to all heads of a token.  A first pass over
    `sample_heads` heads sizes a second one (at most `max_heads`, for memory) to about `target_s` seconds of work
    when the host is fast; the larger sample is the one reported."""
    from oracle import wkv7 as o7

    def one(heads):
        g = np.random.default_rng(1)
        shp = (1, T, heads, N)
        r, k, v = (g.standard_normal(shp) for _ in range(3))
        w = -0.5 + 0.5 * g.standard_normal(shp)
        kap = g.standard_normal(shp)
        kap /= np.linalg.norm(kap, axis=-1, keepdims=True)
        a, b = -kap, kap / (1.0 + np.exp(-g.standard_normal(shp)))
        s = 0.1 * g.standard_normal((1, heads, N, N))
        ns = g.random((1, T)) < 1.0 / 1024
        t0 = time.perf_counter()
        o7.wkv7_assoc_scan(r, w, k, v, a, b, s, np.array([T]), ns, dtype=np.float32)
        return time.perf_counter() - t0

    heads, dt = sample_heads, one(sample_heads)
    if dt < 0.5 * target_s:
        more = min(max_heads, int(np.ceil(sample_heads * target_s / dt)))
        if more > heads:
            heads, dt = more, one(more)
    tok_s = T * (heads / H) / dt
    return {"value": tok_s, "unit": "tokens/s", "cores": threads or (os.cpu_count() or 1), "kind": "port",
            "sample": f"1 sequence, T={T}, {heads} of {H} heads, fp32 log-depth associative scan "
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


def base_record(metric, value, ms_step, args, dtype, workload, extra_config=None):
    cfg = {"workload": workload}
    cfg.update(extra_config or {})
    return {"metric": metric, "value": value, "unit": "tokens/s", "n_gpus": 1, "steps": args.steps,
            "warmup": args.warmup, "ms_per_step": ms_step, "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": dtype, "data": "synthetic", "config": cfg, "prewarm_s": PREWARM_S}


def stream_probe(torch):
    """What a plain streaming kernel reaches on this GPU: torch's c = a + b over three 1 GiB fp32 arrays (two reads
    and one write per element), bytes moved / HIP-event time.  Reported beside the roofline as the practical
    ceiling of the memory system; `roofline.peak` stays the published 8 TB/s."""
    n = (1 << 30) // 4
    a = torch.ones(n, dtype=torch.float32, device="cuda")
    b = torch.ones(n, dtype=torch.float32, device="cuda")
    c = torch.empty(n, dtype=torch.float32, device="cuda")
    for _ in range(3):
        torch.add(a, b, out=c)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(10):
        torch.add(a, b, out=c)
    e1.record()
    torch.cuda.synchronize()
    ms = e0.elapsed_time(e1) / 10
    del a, b, c
    torch.cuda.empty_cache()
    return {"GB/s": 3 * (1 << 30) / (ms * 1e-3) / 1e9, "pattern": "c = a + b, 1 GiB fp32 each (2 reads + 1 write)"}


def roofline(bytes_per_launch, kern_ms, traffic):
    achieved = bytes_per_launch / (kern_ms * 1e-3) / 1e9
    nbytes, source = traffic if traffic is not None else (None, None)
    return {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
            "traffic": nbytes, "traffic_source": source, "kernel_ms": kern_ms, "algorithmic_bytes": bytes_per_launch}


def power_probe(torch, fn, seconds=3.0):
    """Socket power while `fn` runs back to back: the calling thread keeps launching while a second thread waits
    `seconds` / 3 and reads `amd-smi` twice.  None where the tool is missing or prints nothing usable."""
    import shutil
    import subprocess
    import threading
    if shutil.which("amd-smi") is None:
        return None
    got = {"w": [], "done": False}

    def read_power():
        try:
            txt = subprocess.run(["amd-smi", "metric", "-g", "0", "--power"], capture_output=True, text=True, timeout=20).stdout
        except Exception:
            return None
        for line in txt.splitlines():
            if "SOCKET_POWER" in line:
                try:
                    return float(line.split(":")[1].split()[0])
                except (IndexError, ValueError):
                    return None
        return None

    def reader():
        time.sleep(seconds / 3.0)
        got["w"].append(read_power())
        got["w"].append(read_power())
        got["done"] = True

    th = threading.Thread(target=reader)
    th.start()
    while not got["done"]:
        for _ in range(16):
            fn()
        torch.cuda.synchronize()          # keeps the launch queue short, so the loop ends soon after the readings
    th.join()
    cap = None
    try:
        txt = subprocess.run(["rocm-smi", "--showmaxpower"], capture_output=True, text=True, timeout=20).stdout
        for line in txt.splitlines():
            if "Max Graphics Package Power" in line:
                cap = float(line.split(":")[-1])
    except Exception:
        pass
    if all(w is None for w in got["w"]):
        return None
    return {"socket_w": got["w"], "cap_w": cap,
            "how": "amd-smi metric --power, read twice by a second thread while the timed call runs back to back"}


def bench_wkv7(torch, ops, args):
    x = make_inputs(torch)
    tokens = B * T

    def fwd():
        return ops.wkv7_fwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"],
                            compat=True, want_sa=False, force_seq=args.seq)

    wall, kern_ms = time_region(torch, fwd, args.steps, args.warmup)
    ms_step = 1e3 * wall / args.steps
    # r,w,k,v,a,b in + y out (bf16), fp32 state in + out, new_starts, length
    fwd_bytes = 7 * tokens * H * N * 2 + 2 * B * H * N * N * 4 + B * T + B * 4
    out = base_record("WKV7 fwd tokens/s (B8 T4096 H32 N64 bf16)", tokens / (ms_step * 1e-3), ms_step, args, "bf16",
                      "isolated WKV7 op, B=8 T=4096 H=32 N=64, bf16 r/w/k/v/a/b/y, fp32 state, "
                      "new_starts~Bernoulli(1/1024), length~U{T/2..T} (BASELINE configs[1])",
                      {"kernel": "sequential fp32 VALU" if args.seq else "chunked MFMA (fp16 operands, bf16 pairs in the Gram tiles, fp32 state)"})
    out["roofline"] = roofline(fwd_bytes, kern_ms, None if args.seq else measured_traffic("wkv7_fwd"))
    if not args.no_bwd:
        def fwd_bwd():
            new_s, y, sa = ops.wkv7_fwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"],
                                        x["new_starts"], compat=True, want_sa=True, force_seq=args.seq)
            return ops.wkv7_bwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], x["s"], x["length"], x["new_starts"],
                                x["dy"], sa, None, compat=True, force_seq=args.seq)
        n2 = max(10, args.steps // 4)
        wall2, _ = time_region(torch, fwd_bwd, n2, 2)
        ms2 = 1e3 * wall2 / n2
        # forward (7 tensors) + backward reads r,w,k,v,a,b,dy and writes 6 gradients: 20 token tensors in bf16
        fb_bytes = 20 * tokens * H * N * 2 + 4 * B * H * N * N * 4
        out["fwd_bwd"] = {"tokens_per_s": tokens / (ms2 * 1e-3), "ms_per_step": ms2, "steps": n2, "warmup": 2,
                          "hbm_frac": fb_bytes / (ms2 * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": fb_bytes,
                          "note": "forward keeps the residual sa (fp16 beside bf16 I/O); backward = three sweeps (reverse, forward, reverse), " +
                                  ("sequential fp32 VALU kernels" if args.seq else "chunked MFMA kernels") +
                                  "; dsa passes between them as 16-bit fixed point with a scale per 16x16 tile, the decay-gradient terms as fp32 records"}
        if not args.no_power:
            out["fwd_bwd"]["power"] = power_probe(torch, fwd_bwd)
    if not args.no_fp32:
        # the same shape with fp32 r/w/k/v/a/b/y: the chunked kernel on fp32 matrix instructions (or, with --seq, the
        # sequential kernel); 14 token tensors' worth of bytes against the same 8 TB/s
        x32 = {n: (x[n].float() if n in "rwkvab" else x[n]) for n in x}

        def fwd32():
            return ops.wkv7_fwd(x32["r"], x32["w"], x32["k"], x32["v"], x32["a"], x32["b"], x32["s"], x32["length"],
                                x32["new_starts"], compat=True, want_sa=False, force_seq=args.seq)
        n3 = max(2, args.steps // 4)
        _, k32 = time_region(torch, fwd32, n3, 2)
        b32 = 7 * tokens * H * N * 4 + 2 * B * H * N * N * 4 + B * T + B * 4
        out["fp32_io"] = {"tokens_per_s": tokens / (k32 * 1e-3), "kernel_ms": k32,
                          "hbm_frac": b32 / (k32 * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": b32,
                          "mfma_frac": None if args.seq else fp32_mfma_flops(tokens) / (k32 * 1e-3) / 1e12 / 157.3,
                          "kernel": "sequential fp32 VALU" if args.seq else "chunked, v_mfma_f32_16x16x4_f32 (fp32 operands)"}
        if not args.no_bwd:
            # forward (keeping the fp32 residual sa) + the three backward sweeps, all with fp32 I/O
            dy32 = x["dy"].float()

            def fwd_bwd32():
                new_s, y, sa = ops.wkv7_fwd(x32["r"], x32["w"], x32["k"], x32["v"], x32["a"], x32["b"], x32["s"],
                                            x32["length"], x32["new_starts"], compat=True, want_sa=True, force_seq=args.seq)
                return ops.wkv7_bwd(x32["r"], x32["w"], x32["k"], x32["v"], x32["a"], x32["b"], x32["s"], x32["length"],
                                    x32["new_starts"], dy32, sa, None, compat=True, force_seq=args.seq)
            n5 = max(2, args.steps // 10)
            wall5, _ = time_region(torch, fwd_bwd32, n5, 1)
            ms5 = 1e3 * wall5 / n5
            fb32 = 20 * tokens * H * N * 4 + 4 * B * H * N * N * 4
            out["fp32_io"]["fwd_bwd_ms"] = ms5
            out["fp32_io"]["fwd_bwd_tokens_per_s"] = tokens / (ms5 * 1e-3)
            out["fp32_io"]["fwd_bwd_hbm_frac"] = fb32 / (ms5 * 1e-3) / 1e9 / HBM_PEAK_GBS
            # matrix instructions per (chunk, head): forward and sweep A 4 x 80 (consumers) + 96 (producer) each,
            # sweeps B and C 4 x 80 + 64 each; 2048 flop per instruction
            if not args.seq:
                mf = (2 * 416 + 2 * 384) * 2048 * (tokens // 16) * H
                out["fp32_io"]["fwd_bwd_mfma_frac"] = mf / (ms5 * 1e-3) / 1e12 / 157.3
            del dy32
        del x32
    if not args.no_placement and not args.seq:
        # The same two measurements with the seven input arrays copied to addresses 0, 128, ..., 768 bytes past a 1 KiB
        # boundary instead of all on 2 MiB boundaries (where torch's allocator puts them, and where `value` and
        # `fwd_bwd` above are measured): rows of different arrays at the same (token, head) then no longer compete for
        # the same part of the memory system.  A caller that owns the placement of its operands gets these figures.
        xp = dict(x)
        for i, n in enumerate(("r", "w", "k", "v", "a", "b", "dy")):
            xp[n] = ops._empty_phased(tuple(x[n].shape), x[n].dtype, x[n].device, i)
            xp[n].copy_(x[n])

        def fwd_p():
            return ops.wkv7_fwd(xp["r"], xp["w"], xp["k"], xp["v"], xp["a"], xp["b"], xp["s"], xp["length"],
                                xp["new_starts"], compat=True, want_sa=False)

        def fwd_bwd_p():
            new_s, y, sa = ops.wkv7_fwd(xp["r"], xp["w"], xp["k"], xp["v"], xp["a"], xp["b"], xp["s"], xp["length"],
                                        xp["new_starts"], compat=True, want_sa=True)
            return ops.wkv7_bwd(xp["r"], xp["w"], xp["k"], xp["v"], xp["a"], xp["b"], xp["s"], xp["length"],
                                xp["new_starts"], xp["dy"], sa, None, compat=True)
        _, kp = time_region(torch, fwd_p, max(10, args.steps // 2), 3)
        rec = {"inputs_of_value": "every input array on a 2 MiB boundary (torch's allocator); outputs, gradients and "
                                  "workspace arrays at their own 128-byte phases (the operators place them)",
               "inputs_staggered": {"kernel_ms": kp, "tokens_per_s": tokens / (kp * 1e-3),
                                    "hbm_frac": fwd_bytes / (kp * 1e-3) / 1e9 / HBM_PEAK_GBS}}
        if not args.no_bwd:
            n4 = max(10, args.steps // 4)
            wall4, _ = time_region(torch, fwd_bwd_p, n4, 2)
            rec["inputs_staggered"]["fwd_bwd_ms"] = 1e3 * wall4 / n4
        out["placement"] = rec
        del xp
    if not args.no_power:
        out["power"] = power_probe(torch, fwd)
    if args.occupancy_probe:
        # The same kernel on 8, 4 and 2 of the 8 sequences (256, 128, 64 workgroups = CUs): launch time and socket power.
        # Every workgroup does the same work in each case, so a launch time that grows with the number of busy CUs
        # while the socket power approaches its cap shows the power limit (not the kernel's own pipeline) at work.
        probe = []
        for nb in (8, 4, 2):
            xs = {n: (x[n][:nb].contiguous() if n != "dy" else None) for n in x}

            def part():
                return ops.wkv7_fwd(xs["r"], xs["w"], xs["k"], xs["v"], xs["a"], xs["b"], xs["s"], xs["length"],
                                    xs["new_starts"], compat=True, want_sa=False)
            _, kms = time_region(torch, part, 50, 5)
            pw = power_probe(torch, part, seconds=3.0)
            probe.append({"sequences": nb, "workgroups": nb * H, "kernel_ms": kms,
                          "socket_w": None if pw is None else pw["socket_w"]})
        out["occupancy_probe"] = probe
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
        out["cpu_baseline_sequential"] = cpu_baseline_sequential()
        out["gpu_over_cpu"] = out["value"] / out["cpu_baseline"]["value"]
    return out


def fp32_mfma_flops(tokens):
    """Matrix-instruction flops of the fp32 chunked forward: per (16-token chunk, head) the four consumers issue 80
    and the producer 96 v_mfma_f32_16x16x4_f32 of 2*16*16*4 flops each."""
    return tokens / 16 * H * (4 * 80 + 96) * 2 * 16 * 16 * 4


def bench_wkv6(torch, ops, args):
    b6, t6 = 16, 2048
    g = np.random.default_rng(0)
    shp = (b6, t6, H, N)
    f = lambda x: torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).cuda().bfloat16()
    r, k, v, dy = (f(g.standard_normal(shp, dtype=np.float32)) for _ in range(4))
    w = f(-np.exp(-0.5 + 0.5 * g.standard_normal(shp, dtype=np.float32)))
    u = f(0.5 * g.standard_normal((H, N), dtype=np.float32))
    s = torch.zeros((b6, H, N, N), dtype=torch.float32, device="cuda")
    ns = torch.from_numpy(g.random((b6, t6)) < 1.0 / 512).cuda()
    tokens = b6 * t6
    fwd = lambda: ops.wkv6_fwd(r, k, v, w, u, s, None, ns, compat=True)
    wall, kern_ms = time_region(torch, fwd, args.steps, args.warmup)
    ms_step = 1e3 * wall / args.steps
    fwd_bytes = 5 * tokens * H * N * 2 + 2 * b6 * H * N * N * 4 + b6 * t6
    out = base_record("WKV6 fwd tokens/s (B16 T2048 H32 N64 bf16)", tokens / (ms_step * 1e-3), ms_step, args, "bf16",
                      "isolated WKV6 op, B=16 T=2048 H=32 N=64 bf16, zero state, new_starts~Bernoulli(1/512) "
                      "(BASELINE configs[2])",
                      {"kernel": "chunked MFMA; forward on fp16 operands (bf16 pairs in the Gram tile), backward sweeps on "
                                 "bf16 hi+lo pairs; fp32 state and accumulation"})
    out["roofline"] = roofline(fwd_bytes, kern_ms, measured_traffic("wkv6_fwd"))
    if not args.no_bwd:
        fb = lambda: ops.wkv6_bwd(r, k, v, w, u, s, None, ns, dy, None, compat=True)
        n2 = max(10, args.steps // 4)
        wall2, _ = time_region(torch, lambda: (fwd(), fb()), n2, 2)
        ms2 = 1e3 * wall2 / n2
        fb_bytes = 14 * tokens * H * N * 2 + 4 * b6 * H * N * N * 4
        out["fwd_bwd"] = {"tokens_per_s": tokens / (ms2 * 1e-3), "ms_per_step": ms2,
                          "hbm_frac": fb_bytes / (ms2 * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": fb_bytes}
    if not args.no_fp32:
        # the same shape with fp32 r/k/v/w/u/y: the chunked forward on fp32 matrix instructions, and the sequential
        # kernel it replaces for fp32 I/O
        r32, k32, v32, w32, u32 = (t.float() for t in (r, k, v, w, u))
        n3 = max(2, args.steps // 4)
        _, kc = time_region(torch, lambda: ops.wkv6_fwd(r32, k32, v32, w32, u32, s, None, ns, compat=True), n3, 2)
        _, ks = time_region(torch, lambda: ops.wkv6_fwd(r32, k32, v32, w32, u32, s, None, ns, compat=True, force_seq=True), n3, 2)
        b32 = 5 * tokens * H * N * 4 + 2 * b6 * H * N * N * 4 + b6 * t6
        out["fp32_io"] = {"kernel_ms": kc, "tokens_per_s": tokens / (kc * 1e-3),
                          "hbm_frac": b32 / (kc * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": b32,
                          "sequential_kernel_ms": ks, "kernel": "chunked, v_mfma_f32_16x16x4_f32 (fp32 operands)"}
        if not args.no_bwd:
            dy32 = dy.float()

            def fb32(fs):
                ops.wkv6_fwd(r32, k32, v32, w32, u32, s, None, ns, compat=True, force_seq=fs)
                return ops.wkv6_bwd(r32, k32, v32, w32, u32, s, None, ns, dy32, None, compat=True, force_seq=fs)
            n4 = max(2, args.steps // 10)
            wc, _ = time_region(torch, lambda: fb32(False), n4, 1)
            wsq, _ = time_region(torch, lambda: fb32(True), n4, 1)
            out["fp32_io"]["fwd_bwd_ms"] = 1e3 * wc / n4
            out["fp32_io"]["sequential_fwd_bwd_ms"] = 1e3 * wsq / n4
    return out


def bench_wkv4(torch, ops, args):
    b4, t4, c4 = 32, 4096, 2560
    g = np.random.default_rng(0)
    f = lambda x: torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).cuda()
    k = f(g.standard_normal((b4, t4, c4), dtype=np.float32))
    v = f(g.standard_normal((b4, t4, c4), dtype=np.float32))
    w = f(-np.exp(g.standard_normal(c4, dtype=np.float32)))
    u = f(0.5 * g.standard_normal(c4, dtype=np.float32))
    s = torch.zeros((b4, 3, c4), dtype=torch.float32, device="cuda")
    s[:, 2] = -1e38
    length = torch.from_numpy(g.integers(1024, t4 + 1, size=(b4,)).astype(np.int32)).cuda()
    tokens = b4 * t4
    fwd = lambda: ops.wkv4_fwd(w, u, k, v, s, length, None, compat=True)
    wall, kern_ms = time_region(torch, fwd, args.steps, args.warmup)
    ms_step = 1e3 * wall / args.steps
    fwd_bytes = 3 * tokens * c4 * 4 + 2 * b4 * 3 * c4 * 4
    out = base_record("WKV4 fwd tokens/s (B32 T4096 C2560 fp32)", tokens / (ms_step * 1e-3), ms_step, args, "f32",
                      "isolated WKV4 op, B=32 T=4096 C=2560 fp32, state (0,0,-1e38), length~U{1024..4096} "
                      "(BASELINE configs[3])", {"kernel": "one thread per (sequence, channel)"})
    out["roofline"] = roofline(fwd_bytes, kern_ms, measured_traffic("wkv4_fwd"))
    if not args.no_bwd:
        gy = f(g.standard_normal((b4, t4, c4), dtype=np.float32))
        bwd = lambda: ops.wkv4_bwd(w, u, k, v, s, length, None, gy, None, compat=True)
        n2 = max(10, args.steps // 4)
        wall2, kern2 = time_region(torch, bwd, n2, 2)
        # backward alone: reads k, v, gy and writes gk, gv (fp32)
        bwd_bytes = 5 * tokens * c4 * 4
        out["bwd"] = {"ms_per_call": kern2, "hbm_frac": bwd_bytes / (kern2 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                      "algorithmic_bytes": bwd_bytes, "note": "checkpoint pass + reverse pass; workspace and the "
                      "per-sequence gw/gu sums on the host are inside the figure"}

        # training step: the forward keeps the checkpoints, the backward takes them (no checkpoint pass)
        def fwd_bwd():
            _, _, ck = ops.wkv4_fwd(w, u, k, v, s, length, None, compat=True, want_ckpt=True)
            return ops.wkv4_bwd(w, u, k, v, s, length, None, gy, None, compat=True, ckpt=ck)
        _, kern3 = time_region(torch, fwd_bwd, n2, 2)
        fb_bytes = fwd_bytes + bwd_bytes
        out["fwd_bwd"] = {"ms_per_step": kern3, "tokens_per_s": tokens / (kern3 * 1e-3),
                          "hbm_frac": fb_bytes / (kern3 * 1e-3) / 1e9 / HBM_PEAK_GBS, "algorithmic_bytes": fb_bytes,
                          "note": "forward that also writes the state entering every 16th step + reverse pass"}
    return out


def bench_model7(torch, ops, args):
    """BASELINE configs[4]: RWKV-7 1.5B-shaped random-init model through the torch harness with HipRWKV.inner_loop:
    prefill B=16 T=4096 (new_starts ~ Bernoulli(1/2048)) and decode B=256 single-token steps from a carried state."""
    from jaxrwkv_amd.model7 import RWKV7, randomize_weights
    L, C, vocab = 24, 2048, 65536
    bp, tp, bd = 16, 4096, 256
    params = randomize_weights(0, L, C, vocab, dtype=torch.bfloat16, device="cuda", zero_init=True)
    g = torch.Generator(device="cuda")
    g.manual_seed(0)
    tokens = torch.randint(0, vocab, (bp, tp), device="cuda", generator=g)
    ns = torch.rand((bp, tp), device="cuda", generator=g) < 1.0 / 2048
    state = RWKV7.default_state(params, bp)
    steps = max(1, args.steps // 10)

    def prefill():
        with torch.no_grad():
            return RWKV7.forward(params, tokens, state, None, ns)

    wall, _ = time_region(torch, prefill, steps, 1)
    ms_p = 1e3 * wall / steps
    # the recurrence alone at the same shape, all layers
    x = {n: torch.randn((bp, tp, C // N, N), device="cuda", generator=g).bfloat16() for n in ("r", "w", "k", "v", "a", "b")}
    s0 = torch.zeros((bp, C // N, N, N), dtype=torch.bfloat16, device="cuda")
    op = lambda: ops.wkv7_fwd(x["r"], x["w"], x["k"], x["v"], x["a"], x["b"], s0, None, ns, compat=True)
    _, op_ms = time_region(torch, op, 5, 1)
    del x
    # decode
    dtok = torch.randint(0, vocab, (bd, 1), device="cuda", generator=g)
    dstate = (0.1 * torch.randn((bd, L, 2 + N, C), device="cuda", generator=g)).bfloat16()

    def decode():
        with torch.no_grad():
            return RWKV7.forward(params, dtok, dstate, None, None)

    dsteps = max(4, args.steps)
    wall_d, _ = time_region(torch, decode, dsteps, 2)
    ms_d = 1e3 * wall_d / dsteps
    xd = {n: torch.randn((bd, 1, C // N, N), device="cuda", generator=g).bfloat16() for n in ("r", "w", "k", "v", "a", "b")}
    sd = torch.zeros((bd, C // N, N, N), dtype=torch.bfloat16, device="cuda")
    opd = lambda: ops.wkv7_fwd(xd["r"], xd["w"], xd["k"], xd["v"], xd["a"], xd["b"], sd, None, None, compat=True)
    _, opd_ms = time_region(torch, opd, 20, 3)
    # the same decode step replayed from a captured HIP graph (removes the host's launch overhead)
    graph_ms = None
    try:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                decode()
        torch.cuda.current_stream().wait_stream(side)
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            g_logits, g_state = decode()
        torch.cuda.synchronize()
        wall_g, _ = time_region(torch, gr.replay, dsteps, 2)
        graph_ms = 1e3 * wall_g / dsteps
        e_logits, e_state = decode()
        torch.cuda.synchronize()
        graph_ok = bool(torch.equal(g_logits, e_logits) and torch.equal(g_state, e_state))
    except Exception as exc:      # graph capture is an optimisation of the harness, not of the op
        graph_ok = f"capture failed: {type(exc).__name__}: {exc}"[:200]
    out = base_record("RWKV7 1.5B-shaped prefill tokens/s (B16 T4096 bf16, HipRWKV)", bp * tp / (ms_p * 1e-3), ms_p,
                      args, "bf16", "full model L=24 C=2048 H=32 N=64 vocab=65536, bf16 random-init weights, torch "
                      "harness + HipRWKV.inner_loop; prefill B=16 T=4096 new_starts~Bernoulli(1/2048) (BASELINE configs[4])")
    out["steps"], out["warmup"] = steps, 1
    out["prefill"] = {"ms_per_step": ms_p, "wkv_ms_all_layers": L * op_ms, "wkv_fraction": L * op_ms / ms_p}
    out["decode"] = {"tokens_per_s": bd / (ms_d * 1e-3), "ms_per_step": ms_d, "batch": bd,
                     "wkv_ms_all_layers": L * opd_ms, "wkv_fraction": L * opd_ms / ms_d,
                     "hip_graph_ms_per_step": graph_ms,
                     "hip_graph_tokens_per_s": (bd / (graph_ms * 1e-3)) if graph_ms else None,
                     "hip_graph_replay_equals_eager": graph_ok}
    # roofline of the dominant hand-written kernel of this workload: the WKV7 forward at the prefill shape
    tok_heads = bp * tp * (C // N)
    out["roofline"] = roofline(7 * tok_heads * N * 2 + 2 * bp * (C // N) * N * N * 2 + bp * tp, op_ms, None)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--workload", choices=("wkv7", "wkv6", "wkv4", "model7"), default="wkv7")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-bwd", action="store_true")
    ap.add_argument("--no-fp32", action="store_true", help="WKV7: skip the fp32-I/O leg")
    ap.add_argument("--seq", action="store_true", help="WKV7: force the sequential fp32 VALU kernel")
    ap.add_argument("--no-placement", action="store_true", help="skip the run with the inputs at staggered addresses")
    ap.add_argument("--no-power", action="store_true", help="WKV7: skip the socket-power reading (amd-smi)")
    ap.add_argument("--occupancy-probe", action="store_true",
                    help="WKV7: also time the forward on 8, 4 and 2 sequences with a socket-power reading each")
    ap.add_argument("--no-secondary", action="store_true",
                    help="WKV7: skip the compact WKV6 / WKV4 records appended to the line")
    ap.add_argument("--no-stream-probe", action="store_true",
                    help="skip the streaming-bandwidth probe (three 1 GiB arrays) that is reported beside the roofline")
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
    if args.copy_probe:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    out = {"wkv7": bench_wkv7, "wkv6": bench_wkv6, "wkv4": bench_wkv4, "model7": bench_model7}[args.workload](torch, ops, args)
    if args.workload == "wkv7" and not args.no_secondary:
        # the two secondary ops under the same clock: forward time and roofline fraction, forward+backward beside it
        sub = argparse.Namespace(**vars(args))
        sub.steps, sub.warmup = max(20, args.steps // 2), max(3, args.warmup // 2)
        for name, fn in (("wkv6", bench_wkv6), ("wkv4", bench_wkv4)):
            full = fn(torch, ops, sub)
            torch.cuda.empty_cache()
            out[name] = {"workload": full["config"]["workload"], "fwd_ms": full["roofline"]["kernel_ms"],
                         "fwd_tokens_per_s": full["value"], "fwd_hbm_frac": full["roofline"]["frac"],
                         "steps": sub.steps, "warmup": sub.warmup,
                         "fwd_bwd_ms": full.get("fwd_bwd", {}).get("ms_per_step"),
                         "fwd_bwd_hbm_frac": full.get("fwd_bwd", {}).get("hbm_frac")}
    if not args.no_stream_probe:
        out["roofline"]["stream_probe"] = stream_probe(torch)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
