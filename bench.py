#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

A step is one pass of the launch sets that anode's unchanged callers make at
BASELINE.json's configs 1-4 (the "ABI byte model"): u8 cast/dequantize of an
image batch, batch-norm forward (3 launches) and backward (6 launches) at the
two 2-D shapes and the 3-D shape, ReLU forward/backward at the 3-D shape, and
softmax + NLL + backward in row and channel-axis form.  Inputs are synthetic
and resident in HBM before the timed region.  The headline value is
algorithmic bytes of the whole step / wall time of the step.

Prints ONE JSON line.  `roofline` describes the kernel that takes the largest
share of the step, timed with HIP events around each of its launches inside
the timed region; `cpu_baseline` is the CPU restatement of the same kernels
(oracle/, fp32, reference operation order) timed on this host on a bounded
sample of the same workload.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0  # MI355X published HBM3E bandwidth


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--only", default="", help="comma-separated group names to run (default: all)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="add one plain copy of a known size to the step (scale for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    return ap.parse_args()


class Launch:
    """One entry-point call with its algorithmic byte count."""

    def __init__(self, group, symbol, args, alg_bytes, elements):
        self.group, self.symbol, self.args, self.alg_bytes, self.elements = group, symbol, args, alg_bytes, elements


def build_workload(torch, only, copy_calibration=False):
    """All device buffers and the launch list of one step."""
    g = torch.Generator(device="cuda")
    g.manual_seed(0)

    def randn(n, mean=0.0, std=1.0):
        t = torch.randn(n, device="cuda", generator=g)
        if std != 1.0:
            t.mul_(std)
        if mean != 0.0:
            t.add_(mean)
        return t

    def empty(n, dtype=torch.float32):
        return torch.empty(n, device="cuda", dtype=dtype)

    launches = []

    def want(group):
        return not only or group in only

    if copy_calibration:
        n = 64 * 1024 * 1024  # 256 MiB in, 256 MiB out
        src, dst = randn(n), empty(n)
        launches.append(Launch("copy_calibration", "anode_gpu_copy_flat_map_f32", (n, src, dst), 8 * n, n))

    # ---- config 1: u8 image batch [256,3,224,224] -> f32 / u32 -------------------
    if want("cast_cfg1"):
        n = 256 * 3 * 224 * 224
        q = torch.randint(0, 256, (n,), device="cuda", dtype=torch.uint8, generator=g)
        yf, yu = empty(n), empty(n, torch.int32)
        launches.append(Launch("cast_cfg1", "anode_gpu_dequantize_u8_packed_f32", (n, 0.0, 1.0, q, yf), 5 * n, n))
        launches.append(Launch("cast_cfg1", "anode_gpu_upcast_u8_packed_u32", (n, q, yu), 5 * n, n))

    # ---- configs 2a, 2b, 4: batch norm forward + backward -------------------------
    def bn(tag, S, C, N, mean, std):
        n = S * C * N
        x, dy = randn(n, mean, std), randn(n)
        y, dx = empty(n), empty(n)
        m, v, dm, dv = empty(C), empty(C), empty(C), empty(C)
        d = (S, C, N)
        f, b = f"bn_fwd_{tag}", f"bn_bwd_{tag}"
        if want(f) or want(b):
            # forward: mean 4 + var 4 + normalize 8 = 16 B/elem
            launches.append(Launch(f, "anode_gpu_batch_mean_3d1_packed_f32", (*d, x, m), 4 * n, n))
            launches.append(Launch(f, "anode_gpu_batch_var_3d1_packed_f32", (*d, 1e-5, x, m, v), 4 * n, n))
            launches.append(Launch(f, "anode_gpu_batch_norm_3d1_packed_f32", (*d, x, m, v, y), 8 * n, n))
        if want(b):
            # backward: 8 + 4 + 8 + 12 + 4 + 8 = 44 B/elem
            launches.append(Launch(b, "anode_gpu_batch_norm_bwd_3d1_packed_f32", (*d, dy, v, dx), 8 * n, n))
            launches.append(Launch(b, "anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", (*d, dy, v, dm), 4 * n, n))
            launches.append(Launch(b, "anode_gpu_batch_norm_bwd_var_3d1_packed_f32", (*d, dy, x, m, v, dv), 8 * n, n))
            launches.append(Launch(b, "anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", (*d, dv, x, m, dx), 12 * n, n))
            launches.append(Launch(b, "anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", (*d, dv, x, m, dm), 4 * n, n))
            launches.append(Launch(b, "anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", (*d, dm, dx), 8 * n, n))
        return x, dy, y, dx

    bn("cfg2a", 112 * 112, 64, 256, 2.0, 3.0)
    bn("cfg2b", 49, 2048, 256, 2.0, 3.0)
    x4, dy4, y4, dx4 = bn("cfg4", 128 * 128 * 128, 32, 2, 0.0, 1.0)
    if want("relu_cfg4"):
        n = x4.numel()
        # ReLU after BN, in place (examples/bench_unet3d.rs:103), and its mask backward
        launches.append(Launch("relu_cfg4", "anode_gpu_positive_clip_flat_map_f32", (n, y4, y4), 8 * n, n))
        launches.append(Launch("relu_cfg4", "anode_gpu_positive_clip_flat_map_bwd_f32", (n, dy4, y4, dx4), 12 * n, n))

    # ---- config 3a: row softmax + NLL [256,1000] ---------------------------------
    if want("softmax_cfg3a"):
        K, R = 1000, 256
        x = randn(K * R, 0.0, 2.0)
        lab = torch.randint(0, K, (R,), device="cuda", dtype=torch.int32, generator=g)
        p, nll, dx, dy = empty(K * R), empty(R), empty(K * R), torch.ones(R, device="cuda")
        launches.append(Launch("softmax_cfg3a", "anode_gpu_softmax_packed_block_f32", (K, R, x, p), 8 * K * R, K * R))
        launches.append(Launch("softmax_cfg3a", "anode_gpu_softmax_cat_nll_packed_f32", (K, R, p, lab, nll), 12 * R, R))
        launches.append(Launch("softmax_cfg3a", "anode_gpu_softmax_cat_nll_bwd_packed_f32", (K, R, dy, p, lab, dx),
                               8 * K * R + 8 * R, K * R))

    # ---- config 3b: channel-axis softmax + NLL [8,19,512,1024] -------------------
    if want("softmax_cfg3b"):
        P, C, N = 512 * 1024, 19, 8
        n = P * C * N
        x = randn(n)
        lab = torch.randint(0, C, (P * N,), device="cuda", dtype=torch.int32, generator=g)
        lab[torch.rand(P * N, device="cuda", generator=g) < 0.05] = 255
        p, nll, dx, dy = empty(n), empty(P * N), empty(n), torch.ones(P * N, device="cuda")
        launches.append(Launch("softmax_cfg3b", "anode_gpu_softmax_nd_packed_f32", (P, C, N, x, p), 8 * n, n))
        launches.append(Launch("softmax_cfg3b", "anode_gpu_softmax_nd_cat_nll_packed_f32", (P, C, N, p, lab, nll),
                               12 * P * N, P * N))
        launches.append(Launch("softmax_cfg3b", "anode_gpu_softmax_nd_cat_nll_bwd_packed_f32",
                               (P, C, N, dy, p, lab, dx), 8 * n + 8 * P * N, n))
    return launches


def cpu_baseline():
    """The fp32 CPU restatement (reference operation order) on a bounded sample of the same workload."""
    import numpy as np

    from oracle import binding as o

    threads = min(16, os.cpu_count() or 1)
    o.set_threads(threads)
    g = np.random.default_rng(0)
    F32 = np.float32
    total_bytes, total_s = 0, 0.0
    parts = {}

    def timed(name, nbytes, fn):
        nonlocal total_bytes, total_s
        t0 = time.perf_counter()
        fn()
        dt = time.perf_counter() - t0
        total_bytes += nbytes
        total_s += dt
        b, s = parts.get(name, (0, 0.0))
        parts[name] = (b + nbytes, s + dt)

    # batch norm forward + backward on a 64-sample slice of config 2a
    S, C, N = 112 * 112, 64, 64
    n = S * C * N
    x = (2 + 3 * g.standard_normal(n, dtype=np.float32)).astype(F32)
    dy = g.standard_normal(n, dtype=np.float32)
    d = (S, C, N)
    st = {}
    timed("bn", 4 * n, lambda: st.__setitem__("m", o.batch_mean(*d, x)))
    timed("bn", 4 * n, lambda: st.__setitem__("v", o.batch_var(*d, 1e-5, x, st["m"])))
    timed("bn", 8 * n, lambda: o.batch_norm(*d, x, st["m"], st["v"]))
    timed("bn", 8 * n, lambda: st.__setitem__("dx", o.batch_norm_bwd(*d, dy, st["v"])))
    timed("bn", 4 * n, lambda: st.__setitem__("dm", o.batch_norm_bwd_mean(*d, dy, st["v"])))
    timed("bn", 8 * n, lambda: st.__setitem__("dv", o.batch_norm_bwd_var(*d, dy, x, st["m"], st["v"])))
    timed("bn", 12 * n, lambda: st.__setitem__("dx", o.batch_var_bwd(*d, st["dv"], x, st["m"], dx_in=st["dx"])))
    timed("bn", 4 * n, lambda: st.__setitem__("dm", o.batch_var_bwd_mean(*d, st["dv"], x, st["m"], dmean_in=st["dm"])))
    timed("bn", 8 * n, lambda: o.batch_mean_bwd(*d, st["dm"], dx_in=st["dx"]))
    # channel-axis softmax + NLL + backward on four samples of config 3b
    P, C, N = 512 * 1024, 19, 4
    n = P * C * N
    x = g.standard_normal(n, dtype=np.float32)
    lab = g.integers(0, C, P * N).astype(np.uint32)
    timed("softmax_nll", 8 * n, lambda: st.__setitem__("p", o.softmax_nd(P, C, N, x)))
    timed("softmax_nll", 12 * P * N, lambda: o.softmax_nd_cat_nll(P, C, N, st["p"], lab))
    timed("softmax_nll", 8 * n + 8 * P * N, lambda: o.softmax_nd_cat_nll_bwd(P, C, N, np.ones(P * N, F32), st["p"], lab))
    # cast / dequantize on all 256 images of config 1
    n = 256 * 3 * 224 * 224
    q = g.integers(0, 256, n, dtype=np.uint8)
    timed("cast", 5 * n, lambda: o.dequantize_u8(0.0, 1.0, q))
    timed("cast", 5 * n, lambda: o.upcast_u8(q))
    return {
        "value": round(total_bytes / total_s / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": "fp32 CPU restatement, OpenMP: BN fwd+bwd (9 launches) on [64,64,112,112]; softmax_nd+NLL+bwd on "
                  "[4,19,512,1024]; dequantize+upcast on [256,3,224,224]; algorithmic bytes / time",
        "parts_gbps": {k: round(b / s / 1e9, 3) for k, (b, s) in parts.items()},
        "seconds": round(total_s, 2),
    }


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py: this build measures one GPU; --gpus above 1 is not supported\n")
        sys.exit(2)
    import torch

    from anode_amd import gpu

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        sys.exit(3)
    torch.cuda.set_device(0)
    only = set(filter(None, args.only.split(",")))
    launches = build_workload(torch, only, args.copy_calibration)
    torch.cuda.synchronize()

    def run_step(wrap_symbol=None, events=None):
        for l in launches:
            if wrap_symbol is not None and l.symbol == wrap_symbol[0] and l.group == wrap_symbol[1]:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                gpu.call(l.symbol, *l.args)
                b.record()
                events.append((a, b))
            else:
                gpu.call(l.symbol, *l.args)

    # warm-up (also grows the library's scratch buffers outside the timed region)
    for _ in range(max(1, args.warmup)):
        run_step()
    torch.cuda.synchronize()
    assert gpu.take_last_error() == 0

    # untimed calibration pass: per-launch HIP-event durations for the breakdown
    per_launch = [[] for _ in launches]
    for _ in range(3):
        evs = []
        for l in launches:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            gpu.call(l.symbol, *l.args)
            b.record()
            evs.append((a, b))
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(evs):
            per_launch[i].append(a.elapsed_time(b) * 1e-3)
    med = [sorted(t)[len(t) // 2] for t in per_launch]
    dom_i = max(range(len(launches)), key=lambda i: med[i])
    dom = launches[dom_i]

    # timed region: exactly K steps between synchronisations
    events = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        run_step((dom.symbol, dom.group), events)
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    assert gpu.take_last_error() == 0
    step_s = (t1 - t0) / args.steps
    step_bytes = sum(l.alg_bytes for l in launches)
    step_elems = sum(l.elements for l in launches)
    value = step_bytes / step_s / 1e9

    dom_s = sum(a.elapsed_time(b) for a, b in events) * 1e-3 / len(events)
    roofline = {
        "bound": "hbm",
        "kernel": dom.symbol,
        "workload": dom.group,
        "achieved": round(dom.alg_bytes / dom_s / 1e9, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(dom.alg_bytes / dom_s / 1e9 / HBM_PEAK_GBPS, 4),
        "alg_bytes_per_launch": dom.alg_bytes,
        "avg_launch_us": round(dom_s * 1e6, 2),
        "traffic": None,
    }

    groups = {}
    for l, t in zip(launches, med):
        b, s, e = groups.get(l.group, (0, 0.0, 0))
        groups[l.group] = (b + l.alg_bytes, s + t, e + l.elements)
    breakdown = {k: {"gbps": round(b / s / 1e9, 1), "pct_of_peak": round(100 * b / s / 1e9 / HBM_PEAK_GBPS, 1),
                     "us": round(s * 1e6, 1), "gelem_per_s": round(e / s / 1e9, 2)} for k, (b, s, e) in groups.items()}
    per_symbol = [{"group": l.group, "symbol": l.symbol.replace("anode_gpu_", ""), "us": round(t * 1e6, 1),
                   "gbps": round(l.alg_bytes / t / 1e9, 1)} for l, t in zip(launches, med)]

    out = {
        "metric": "achieved HBM GB/s & % of peak: BN fwd/bwd, softmax-NLL, quantize/cast",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(step_s * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": "configs[1..4], ABI byte model: cast+dequantize u8[256,3,224,224]; BN fwd(3)+bwd(6 launches) "
                        "f32 [256,64,112,112], [256,2048,7,7], [2,32,128,128,128] + ReLU fwd/bwd; softmax+NLL+bwd "
                        "[256,1000] and [8,19,512,1024]",
            "launches_per_step": len(launches),
            "alg_bytes_per_step": step_bytes,
        },
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "gelem_per_s": round(step_elems / step_s / 1e9, 2),
        "roofline": roofline,
        "breakdown": breakdown,
        "per_symbol": per_symbol,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline()
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
