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
    ap.add_argument("--stream-probe", action="store_true",
                    help="instead of the benchmark: time the library's plain copy and a read-only reduction on cold "
                         "822 MB arrays under the launch-geometry and cache-policy knobs, one JSON line")
    ap.add_argument("--all-symbols", action="store_true",
                    help="instead of the benchmark: every entry point once at a bandwidth-sized shape, one JSON line")
    ap.add_argument("--shape-sweep", action="store_true",
                    help="instead of the benchmark: batch-norm pieces over S x C, row softmax over K and channel-axis "
                         "softmax over C x P, each on ~256 MB arrays, one JSON line (where the tilings switch)")
    ap.add_argument("--offset-views", action="store_true",
                    help="instead of the benchmark: the configs' dominant entry points with arrays on 16-byte "
                         "boundaries, one element past them, and 1, 2, 3 elements past them, one JSON line")
    ap.add_argument("--source-fingerprints", action="store_true",
                    help="print the fingerprints of the kernel sources behind the measured-traffic table and exit")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="add one plain copy of a known size to the step (scale for rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    return ap.parse_args()


class Launch:
    """One entry-point call with its algorithmic byte count."""

    def __init__(self, group, symbol, args, alg_bytes, elements):
        self.group, self.symbol, self.args, self.alg_bytes, self.elements = group, symbol, args, alg_bytes, elements


# HBM bytes per launch from hardware counters, keyed by (symbol, workload group): two rocprofv3 --pmc runs of this
# file (FETCH_SIZE, then WRITE_SIZE, KiB per dispatch), each scaled by what the same counter reads for a plain copy
# of known size in the same run (--copy-calibration): FETCH_SIZE x 2.000, WRITE_SIZE x 1.000.  These are the figures
# of the profile named in TRAFFIC_SOURCE, not re-measured by this run; a launch that is not listed reports null.
TRAFFIC_SOURCE = "profiles/bench_step_dominant_kernels_hbm_traffic.md (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, not re-measured in this run)"
MEASURED_TRAFFIC = {
    ("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", "bn_bwd_cfg2a"): (2466157832, "bn_maps"),
    ("anode_gpu_batch_norm_3d1_packed_f32", "bn_fwd_cfg2a"): (1644153473, "bn_maps"),
    ("anode_gpu_batch_mean_3d1_packed_f32", "bn_fwd_cfg2b"): (102823499, "bn_reductions"),
    ("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", "bn_bwd_cfg2b"): (205591707, "bn_reductions"),
    ("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", "bn_bwd_cfg2b"): (308434067, "bn_maps"),
    ("anode_gpu_positive_clip_flat_map_bwd_f32", "relu_cfg4"): (1610547205, "flat_maps"),
    ("anode_gpu_softmax_nd_packed_f32", "softmax_cfg3b"): (637597563, "softmax"),
    ("anode_gpu_softmax_nd_cat_nll_packed_f32", "softmax_cfg3b"): (291407352, "softmax"),
    ("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", "softmax_cfg3b"): (671288431, "softmax"),
    ("anode_gpu_dequantize_u8_packed_f32", "cast_cfg1"): (192699228, "flat_maps"),
    ("anode_gpu_upcast_u8_packed_u32", "cast_cfg1"): (192703324, "flat_maps"),
}
# The kernel sources behind each family of the table and their fingerprint when the counters were read (sha256 over
# the files' bytes, first 16 hex digits).  A figure whose family's sources have changed since is reported as null
# with a note instead of the stale number: run the two counter passes again, update the table and the fingerprints
# (`python3 bench.py --source-fingerprints` prints the current ones).
TRAFFIC_FAMILY_SOURCES = {
    "bn_maps": ["common.hpp", "chan_map.hpp", "batch_norm.hip"],
    "bn_reductions": ["common.hpp", "chan_reduce.hpp", "batch_norm.hip"],
    "flat_maps": ["common.hpp", "flat_map.hip"],
    "softmax": ["common.hpp", "softmax.hip"],
}
TRAFFIC_FAMILY_FINGERPRINT = {
    "bn_maps": "9d94a1d3c0e0f479",
    "bn_reductions": "e27eb3a6158f909f",
    "flat_maps": "c8b36a639e6d43e9",
    "softmax": "a3e766a866176ae6",
}


def source_fingerprints():
    import hashlib
    here = os.path.join(os.path.dirname(os.path.abspath(__file__)), "anode_amd", "csrc")
    out = {}
    for family, files in TRAFFIC_FAMILY_SOURCES.items():
        h = hashlib.sha256()
        try:
            for f in files:
                with open(os.path.join(here, f), "rb") as fh:
                    h.update(fh.read())
            out[family] = h.hexdigest()[:16]
        except OSError:
            out[family] = None
    return out


def measured_traffic(symbol, group, current):
    """(bytes or None, note or None) for a launch of the table; None/None for a launch that is not in it."""
    entry = MEASURED_TRAFFIC.get((symbol, group))
    if entry is None:
        return None, None
    nbytes, family = entry
    if current.get(family) != TRAFFIC_FAMILY_FINGERPRINT.get(family):
        return None, (f"STALE: the sources of the {family} kernels ({', '.join(TRAFFIC_FAMILY_SOURCES[family])}) have changed "
                      f"since the counters were read ({nbytes} bytes then); the counter passes must be repeated")
    return nbytes, None


class Draws:
    """Synthetic inputs drawn as the measurement spec prescribes: numpy.random.default_rng(0) (PCG64), normals and
    uniforms drawn in float64 and cast to float32, labels from integers(); one generator for the whole workload,
    consumed in the order configs 1, 2a, 2b, 3a, 3b, 4 (within a config: the order the arrays are listed in
    `config.inputs`).  Arrays are produced in chunks so that an 822 MB tensor never needs its float64 image on the
    host at once."""

    CHUNK = 1 << 24

    def __init__(self, torch, np):
        self.torch, self.np = torch, np
        self.rng = np.random.default_rng(0)

    def _fill(self, out, make):
        n = out.numel()
        for lo in range(0, n, self.CHUNK):
            m = min(self.CHUNK, n - lo)
            out[lo:lo + m].copy_(self.torch.from_numpy(make(m)))
        return out

    def normal(self, out, mean=0.0, std=1.0):
        np = self.np
        return self._fill(out, lambda m: (mean + std * self.rng.standard_normal(m)).astype(np.float32))

    def uniform(self, out, lo, hi):
        np = self.np
        return self._fill(out, lambda m: (lo + (hi - lo) * self.rng.random(m)).astype(np.float32))

    def integers(self, out, hi):
        np = self.np
        if out.dtype == self.torch.uint8:
            return self._fill(out, lambda m: self.rng.integers(0, hi, m, dtype=np.uint8))
        return self._fill(out, lambda m: self.rng.integers(0, hi, m).astype(np.uint32).view(np.int32))

    def mask(self, n, prob):
        out = self.torch.empty(n, device="cuda", dtype=self.torch.bool)
        return self._fill(out, lambda m: self.rng.random(m) < prob)


def build_workload(torch, only, copy_calibration=False):
    """All device buffers and the launch list of one step."""
    import numpy as np

    draw = Draws(torch, np)

    def empty(n, dtype=torch.float32):
        return torch.empty(n, device="cuda", dtype=dtype)

    launches = []
    fused = []  # additive entry points on the same buffers (fused byte model); measured beside the step, not in it

    def want(group):
        return not only or group in only

    if copy_calibration:
        n = 64 * 1024 * 1024  # 256 MiB in, 256 MiB out
        src, dst = torch.randn(n, device="cuda"), empty(n)
        launches.append(Launch("copy_calibration", "anode_gpu_copy_flat_map_f32", (n, src, dst), 8 * n, n))

    # ---- device arrays are allocated in launch order (config 1, 2a, 2b, 4, 3a, 3b: x, dy, y, dx per layer) and then
    # ---- filled by draws in config order (1, 2a, 2b, 3a, 3b, 4)
    n1 = 256 * 3 * 224 * 224
    cast = want("cast_cfg1")
    q1 = empty(n1, torch.uint8) if cast else None
    yf1, yu1 = (empty(n1), empty(n1, torch.int32)) if cast else (None, None)
    z1, zq1 = (empty(n1), empty(n1, torch.uint8)) if cast else (None, None)
    bn_shapes = {"cfg2a": (112 * 112, 64, 256, 2.0, 3.0), "cfg2b": (49, 2048, 256, 2.0, 3.0),
                 "cfg4": (128 * 128 * 128, 32, 2, 0.0, 1.0)}
    bn_data = {}
    for tag, (S, C, N, _, _) in bn_shapes.items():
        if want(f"bn_fwd_{tag}") or want(f"bn_bwd_{tag}") or (tag == "cfg4" and want("relu_cfg4")):
            n = S * C * N
            bn_data[tag] = {"x": empty(n), "dy": empty(n), "y": empty(n), "dx": empty(n),
                            "gamma": torch.ones(C, device="cuda"), "beta": torch.zeros(C, device="cuda")}
    sm3a = sm3b = None
    if want("softmax_cfg3a"):
        sm3a = (empty(1000 * 256), empty(256, torch.int32))
    if want("softmax_cfg3b"):
        sm3b = (empty(512 * 1024 * 19 * 8), empty(512 * 1024 * 8, torch.int32))

    if cast:
        draw.integers(q1, 256)
        draw.normal(z1)
    for tag in ("cfg2a", "cfg2b"):
        if tag in bn_data:
            _, _, _, mean, std = bn_shapes[tag]
            draw.normal(bn_data[tag]["x"], mean, std)
            draw.normal(bn_data[tag]["dy"])
            draw.uniform(bn_data[tag]["gamma"], 0.5, 1.5)
            draw.normal(bn_data[tag]["beta"], 0.0, 0.1)
    if sm3a is not None:
        draw.normal(sm3a[0], 0.0, 2.0)          # "N(0,4)": variance 4, sigma 2
        draw.integers(sm3a[1], 1000)
    if sm3b is not None:
        draw.normal(sm3b[0])
        draw.integers(sm3b[1], 19)
        sm3b[1][draw.mask(512 * 1024 * 8, 0.05)] = 255   # 5 % ignore-index
    if "cfg4" in bn_data:                        # gamma = 1, beta = 0
        draw.normal(bn_data["cfg4"]["x"])
        draw.normal(bn_data["cfg4"]["dy"])

    # ---- config 1: u8 image batch [256,3,224,224] -> f32 / u32 -------------------
    if want("cast_cfg1"):
        n, yf, yu, zq = n1, yf1, yu1, zq1
        launches.append(Launch("cast_cfg1", "anode_gpu_dequantize_u8_packed_f32", (n, 0.0, 1.0, q1, yf), 5 * n, n))
        launches.append(Launch("cast_cfg1", "anode_gpu_upcast_u8_packed_u32", (n, q1, yu), 5 * n, n))
        # what the config names beyond the reference's two casts: per-channel image normalisation in one pass, and
        # f32 -> u8 quantisation of an N(0,1) tensor (scale 8/255, zero point at -4; parity unpinned by the
        # reference, which has no such kernel)
        a = torch.tensor([1 / (255 * 0.229), 1 / (255 * 0.224), 1 / (255 * 0.225)], device="cuda")
        b = torch.tensor([-0.485 / 0.229, -0.456 / 0.224, -0.406 / 0.225], device="cuda")
        fused.append(Launch("fused_cast_cfg1", "anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32",
                            (224 * 224, 3, 256, a, b, q1, yf), 5 * n, n))
        fused.append(Launch("fused_cast_cfg1", "anode_gpu_quantize_u8_packed_f32", (n, -4.0, 4.0, z1, zq), 5 * n, n))

    # ---- configs 2a, 2b, 4: batch norm forward + backward -------------------------
    def bn(tag, relu=False):
        if tag not in bn_data:
            return None
        S, C, N, _, _ = bn_shapes[tag]
        t = bn_data[tag]
        x, dy, y, dx, gamma, beta = t["x"], t["dy"], t["y"], t["dx"], t["gamma"], t["beta"]
        n = S * C * N
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
        if want(f) or want(b):
            # fused byte model: forward 4 + 8 = 12 B/elem; backward 8 + 12 = 20 B/elem (with the ReLU mask 12 + 16)
            y2, dx2, m2, v2, dm2, dv2 = empty(n), empty(n), empty(C), empty(C), empty(C), empty(C)
            norm = "anode_gpu_batch_norm_positive_clip_3d1_packed_f32" if relu else "anode_gpu_batch_norm_3d1_packed_f32"
            fused.append(Launch(f"fused_{f}", "anode_gpu_batch_mean_var_3d1_packed_f32", (*d, 1e-5, x, m2, v2), 4 * n, n))
            fused.append(Launch(f"fused_{f}", norm, (*d, x, m2, v2, y2), 8 * n, n))
            mask = y2 if relu else None
            fused.append(Launch(f"fused_{b}", "anode_gpu_batch_norm_bwd_reduce_3d1_packed_f32",
                                (*d, dy, x, m2, v2, mask, dm2, dv2), (12 if relu else 8) * n, n))
            fused.append(Launch(f"fused_{b}", "anode_gpu_batch_norm_bwd_apply_3d1_packed_f32",
                                (*d, dy, x, m2, v2, dm2, dv2, mask, dx2), (16 if relu else 12) * n, n))
            if not relu:
                # the layer the config words: batch statistics, normalise with gamma / beta, running statistics with
                # momentum 0.1 (src/ops.rs:1002-1003: online_average of the mean and of var + eps)
                rm, rv = torch.zeros(C, device="cuda"), torch.ones(C, device="cuda")
                g_ = f"affine_{f}"
                fused.append(Launch(g_, "anode_gpu_batch_mean_var_3d1_packed_f32", (*d, 1e-5, x, m2, v2), 4 * n, n))
                fused.append(Launch(g_, "anode_gpu_batch_norm_affine_3d1_packed_f32", (*d, x, m2, v2, gamma, beta, y2), 8 * n, n))
                fused.append(Launch(g_, "anode_gpu_online_average_packed_f32", (C, 0.1, m2, rm), 12 * C, C))
                fused.append(Launch(g_, "anode_gpu_online_average_packed_f32", (C, 0.1, v2, rv), 12 * C, C))
                # the same layer with the running statistics moved by the statistics launch itself
                rm2, rv2 = torch.zeros(C, device="cuda"), torch.ones(C, device="cuda")
                g2_ = f"affine_one_stats_launch_{f}"
                fused.append(Launch(g2_, "anode_gpu_batch_mean_var_online_3d1_packed_f32",
                                    (*d, 1e-5, 0.1, x, m2, v2, rm2, rv2), 4 * n + 24 * C, n))
                fused.append(Launch(g2_, "anode_gpu_batch_norm_affine_3d1_packed_f32", (*d, x, m2, v2, gamma, beta, y2), 8 * n, n))
        return x, dy, y, dx

    bn("cfg2a")
    bn("cfg2b")
    r4 = bn("cfg4", relu=True)
    if want("relu_cfg4") and r4 is not None:
        x4, dy4, y4, dx4 = r4
        n = x4.numel()
        # ReLU after BN, in place (examples/bench_unet3d.rs:103), and its mask backward
        launches.append(Launch("relu_cfg4", "anode_gpu_positive_clip_flat_map_f32", (n, y4, y4), 8 * n, n))
        launches.append(Launch("relu_cfg4", "anode_gpu_positive_clip_flat_map_bwd_f32", (n, dy4, y4, dx4), 12 * n, n))

    # ---- config 3a: row softmax + NLL [256,1000] ---------------------------------
    if sm3a is not None:
        K, R = 1000, 256
        x, lab = sm3a
        p, nll, dx, dy = empty(K * R), empty(R), empty(K * R), torch.ones(R, device="cuda")
        launches.append(Launch("softmax_cfg3a", "anode_gpu_softmax_packed_block_f32", (K, R, x, p), 8 * K * R, K * R))
        launches.append(Launch("softmax_cfg3a", "anode_gpu_softmax_cat_nll_packed_f32", (K, R, p, lab, nll), 12 * R, R))
        launches.append(Launch("softmax_cfg3a", "anode_gpu_softmax_cat_nll_bwd_packed_f32", (K, R, dy, p, lab, dx),
                               8 * K * R + 8 * R, K * R))
        p2, nll2, dx2 = empty(K * R), empty(R), empty(K * R)
        fused.append(Launch("fused_softmax_cfg3a", "anode_gpu_softmax_cat_nll_fused_packed_f32",
                            (K, R, x, lab, p2, nll2), 8 * K * R + 8 * R, K * R))
        fused.append(Launch("fused_softmax_cfg3a", "anode_gpu_softmax_cat_nll_bwd_packed_f32", (K, R, dy, p2, lab, dx2),
                            8 * K * R + 8 * R, K * R))

        p3, nll3, dx3 = empty(K * R), empty(R), empty(K * R)
        fused.append(Launch("fused_softmax_fwd_bwd_cfg3a", "anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32",
                            (K, R, x, lab, dy, p3, nll3, dx3), 12 * K * R + 12 * R, K * R))

    # ---- config 3b: channel-axis softmax + NLL [8,19,512,1024] -------------------
    if sm3b is not None:
        P, C, N = 512 * 1024, 19, 8
        n = P * C * N
        x, lab = sm3b
        p, nll, dx, dy = empty(n), empty(P * N), empty(n), torch.ones(P * N, device="cuda")
        launches.append(Launch("softmax_cfg3b", "anode_gpu_softmax_nd_packed_f32", (P, C, N, x, p), 8 * n, n))
        launches.append(Launch("softmax_cfg3b", "anode_gpu_softmax_nd_cat_nll_packed_f32", (P, C, N, p, lab, nll),
                               12 * P * N, P * N))
        launches.append(Launch("softmax_cfg3b", "anode_gpu_softmax_nd_cat_nll_bwd_packed_f32",
                               (P, C, N, dy, p, lab, dx), 8 * n + 8 * P * N, n))
        p2, nll2 = empty(n), empty(P * N)
        fused.append(Launch("fused_softmax_fwd_cfg3b", "anode_gpu_softmax_nd_cat_nll_fused_packed_f32",
                            (P, C, N, x, lab, p2, nll2), 8 * n + 8 * P * N, n))
        # forward and backward in one launch for the dy of a summed loss: x, labels, dy in; p, nll, dx out
        dx2 = empty(n)
        fused.append(Launch("fused_softmax_fwd_bwd_cfg3b", "anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32",
                            (P, C, N, x, lab, dy, p2, nll2, dx2), 12 * n + 12 * P * N, n))
    return launches, fused


def stream_probe(torch, gpu):
    """The two measurements behind the launch geometry and the cache policy of the streaming kernels."""
    n = 205520896  # 822 MB of f32
    pairs = [(torch.randn(n, device="cuda"), torch.empty(n, device="cuda")) for _ in range(4)]  # rotate: cold data
    S, C, N = 12544, 64, 256
    mean = torch.empty(C, device="cuda")

    def rate(fn, nbytes, reps=12):
        for i in range(2):
            fn(i)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(reps):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return round(nbytes / (a.elapsed_time(b) * 1e-3 / reps) / 1e9, 1)

    saved = [gpu.set_tuning(k, -1) for k in range(6)]
    out = {"bytes_per_array": 4 * n, "copy_gbps": {}, "batch_mean_gbps": {}}
    gpu.set_tuning(5, 0)
    for wg in (0, 8, 32):
        for nt in (0, 3):
            gpu.set_tuning(0, wg)
            gpu.set_tuning(3, nt)
            key = f"{'full_grid' if wg == 0 else str(wg) + '_wg_per_cu'}_{'nontemporal' if nt else 'default'}"
            out["copy_gbps"][key] = rate(lambda i: gpu.call("anode_gpu_copy_flat_map_f32", n, *pairs[i % 4]), 8 * n)
    for rnt in (0, 2):
        gpu.set_tuning(4, rnt)
        key = "nontemporal" if rnt else "default"
        out["batch_mean_gbps"][key] = rate(
            lambda i: gpu.call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, pairs[i % 4][0], mean), 4 * n)
    for k, v in enumerate(saved):
        gpu.set_tuning(k, v)
    del pairs
    torch.cuda.empty_cache()

    # What a plane-strided walk costs at config 3b, [8,19,512,1024] (319 MB arrays), library defaults: a flat copy,
    # the n-d NLL backward (reads one plane and writes one plane at a time: no dependency between planes), and the n-d
    # softmax (all 19 planes of a pixel group must have arrived before the first can be stored), each from cold arrays.
    P, Cc, Nn = 512 * 1024, 19, 8
    m = P * Cc * Nn
    sets = [(torch.randn(m, device="cuda"), torch.empty(m, device="cuda")) for _ in range(3)]
    lab = torch.randint(0, Cc, (P * Nn,), device="cuda", dtype=torch.int32)
    ones = torch.ones(P * Nn, device="cuda")
    out["planes_319MB_gbps"] = {
        "flat_copy": rate(lambda i: gpu.call("anode_gpu_copy_flat_map_f32", m, *sets[i % 3]), 8 * m),
        "softmax_nd_cat_nll_bwd (plane by plane)": rate(
            lambda i: gpu.call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, Cc, Nn, ones, sets[i % 3][0], lab,
                               sets[i % 3][1]), 8 * m + 8 * P * Nn),
        "softmax_nd (all planes, then store)": rate(
            lambda i: gpu.call("anode_gpu_softmax_nd_packed_f32", P, Cc, Nn, *sets[i % 3]), 8 * m),
    }
    del sets
    torch.cuda.empty_cache()

    def one(fn):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        fn()
        b.record()
        torch.cuda.synchronize()
        return a.elapsed_time(b) * 1e-3

    # What the launch before it does to a kernel: dequantize of u8 [256,3,224,224] (38.5 MB in, 154 MB out) right
    # after a reader (batch_mean over 822 MB) and right after a writer (copy of 822 MB), library defaults.
    nq = 256 * 3 * 224 * 224
    q = torch.randint(0, 256, (nq,), device="cuda", dtype=torch.uint8)
    yq = torch.empty(nq, device="cuda")
    Sb, Cb, Nb = 12544, 64, 256
    big = torch.randn(Sb * Cb * Nb, device="cuda")
    bigdst = torch.empty(Sb * Cb * Nb, device="cuda")
    mean = torch.empty(Cb, device="cuda")
    after_reader, after_writer = [], []
    for _ in range(8):
        gpu.call("anode_gpu_batch_mean_3d1_packed_f32", Sb, Cb, Nb, big, mean)
        after_reader.append(one(lambda: gpu.call("anode_gpu_dequantize_u8_packed_f32", nq, 0.0, 1.0, q, yq)))
        gpu.call("anode_gpu_copy_flat_map_f32", big.numel(), big, bigdst)
        after_writer.append(one(lambda: gpu.call("anode_gpu_dequantize_u8_packed_f32", nq, 0.0, 1.0, q, yq)))
    med = lambda t: sorted(t[1:])[len(t[1:]) // 2]  # noqa: E731
    out["dequantize_cfg1_us"] = {"after_a_reader_of_822MB": round(med(after_reader) * 1e6, 1),
                                 "after_a_writer_of_822MB": round(med(after_writer) * 1e6, 1)}
    return out


def shape_sweep(torch, gpu):
    """Bandwidth of the main kernel families across the shapes at which their tilings switch (algorithmic bytes /
    time of 8 launches in rotation over cold arrays).  Every array handed to an entry point is a view of exactly the
    element count the dims describe, checked before the call."""
    total = 64 << 20  # elements per buffer (256 MB of f32)
    bufs = [torch.randn(total, device="cuda") for _ in range(6)]
    labels = torch.zeros(total, device="cuda", dtype=torch.int32)

    def rate(fn, nbytes, reps=8):
        for i in range(2):
            fn(i)
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        for i in range(reps):
            fn(i)
        b.record()
        torch.cuda.synchronize()
        return round(nbytes / (a.elapsed_time(b) * 1e-3 / reps) / 1e9)

    def views(n):
        assert 0 < n <= total
        v = [b[:n] for b in bufs]
        assert all(t.numel() == n for t in v)
        return v

    out = {"elements_per_array_at_most": total, "unit": "GB/s of algorithmic bytes", "batch_norm": [], "row_softmax": [],
           "nd_softmax": []}
    for S in (1, 2, 4, 7, 16, 49, 64, 196, 256, 257, 784, 1024, 1025, 3136, 4096, 4097, 12544, 200704):
        for C in (4, 64, 2048):
            if S * C > total:
                continue
            N = min(total // (S * C), 1 << 20)
            n = S * C * N
            x = views(n)
            mean, var, red = (torch.zeros(C, device="cuda"), torch.ones(C, device="cuda"), torch.empty(C, device="cuda"))
            out["batch_norm"].append({
                "S": S, "C": C, "N": N,
                "batch_mean": rate(lambda i: gpu.call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, x[i % 3], red), 4 * n),
                "batch_norm_bwd_var": rate(lambda i: gpu.call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", S, C, N,
                                                              x[i % 3], x[3 + i % 3], mean, var, red), 8 * n),
                "batch_norm": rate(lambda i: gpu.call("anode_gpu_batch_norm_3d1_packed_f32", S, C, N, x[i % 3], mean, var,
                                                      x[3 + i % 3]), 8 * n),
                "batch_var_bwd_accumulate": rate(lambda i: gpu.call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32",
                                                                    S, C, N, var, x[i % 3], mean, x[3 + i % 3]), 12 * n)})
    for K in (8, 10, 19, 32, 33, 64, 100, 128, 200, 224, 232, 240, 256, 512, 1000, 1024, 2048, 2049, 4096, 16384, 16385,
              32768, 32772, 50000, 50257, 65536, 262144):
        R = total // K
        n = K * R
        x = views(n)
        out["row_softmax"].append({
            "K": K, "R": R,
            "softmax_packed_block": rate(lambda i: gpu.call("anode_gpu_softmax_packed_block_f32", K, R, x[i % 3],
                                                            x[3 + i % 3]), 8 * n)})
    for P in (65536, 4225, 400, 196):
        for C in (2, 4, 19, 32, 33, 64, 100, 128, 150, 256, 300):
            N = min(total // (P * C), 1 << 20)
            if N < 1:
                continue
            n = P * C * N
            x = views(n)
            lab, dy = labels[:P * N], bufs[5][:P * N]
            assert lab.numel() == P * N and dy.numel() == P * N
            out["nd_softmax"].append({
                "P": P, "C": C, "N": N,
                "softmax_nd": rate(lambda i: gpu.call("anode_gpu_softmax_nd_packed_f32", P, C, N, x[i % 2], x[2 + i % 2]),
                                   8 * n),
                "softmax_nd_cat_nll_bwd": rate(lambda i: gpu.call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dy,
                                                                  x[i % 2], lab, x[2 + i % 2]), 8 * n)})
    return out


def all_symbols(torch, gpu):
    """Every entry point of the reference ABI (and the additive ones) once, at a bandwidth-sized shape: median time
    of 50 launches made in rotation with the others (so each launch meets a cold cache), algorithmic bytes / time."""
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    E = lambda n, dt=torch.float32: torch.empty(n, device="cuda", dtype=dt)  # noqa: E731
    Rn = lambda n: torch.randn(n, device="cuda", generator=g)                # noqa: E731
    L = []

    def add(symbol, shape, args, nbytes):
        L.append((symbol, shape, args, nbytes))

    # batch-norm family on [256,64,112,112]
    S, C, N = 112 * 112, 64, 256
    n = S * C * N
    d = (S, C, N)
    x, dy, y, dx = Rn(n), Rn(n), E(n), Rn(n)
    m, v, dm, dv = Rn(C), torch.rand(C, device="cuda", generator=g) + 0.5, Rn(C), Rn(C)
    sh = "[256,64,112,112]"
    add("anode_gpu_batch_mean_3d1_packed_f32", sh, (*d, x, E(C)), 4 * n)
    add("anode_gpu_batch_var_3d1_packed_f32", sh, (*d, 1e-5, x, m, E(C)), 4 * n)
    add("anode_gpu_batch_norm_3d1_packed_f32", sh, (*d, x, m, v, y), 8 * n)
    add("anode_gpu_batch_norm_bwd_3d1_packed_f32", sh, (*d, dy, v, y), 8 * n)
    add("anode_gpu_batch_norm_bwd_3d1_packed_accumulate_f32", sh, (*d, dy, v, dx), 12 * n)
    add("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", sh, (*d, dy, v, E(C)), 4 * n)
    add("anode_gpu_batch_norm_bwd_mean_3d1_packed_accumulate_f32", sh, (*d, dy, v, dm), 4 * n)
    add("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", sh, (*d, dy, x, m, v, E(C)), 8 * n)
    add("anode_gpu_batch_norm_bwd_var_3d1_packed_accumulate_f32", sh, (*d, dy, x, m, v, dv), 8 * n)
    add("anode_gpu_batch_norm_bwd_var_v2_3d1_packed_f32", sh, (*d, dy, x, v, E(C)), 8 * n)
    add("anode_gpu_batch_norm_bwd_var_v2_3d1_packed_accumulate_f32", sh, (*d, dy, x, v, dv), 8 * n)
    add("anode_gpu_batch_var_bwd_3d1_packed_f32", sh, (*d, dv, x, m, y), 8 * n)
    add("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", sh, (*d, dv, x, m, dx), 12 * n)
    add("anode_gpu_batch_var_bwd_mean_3d1_packed_f32", sh, (*d, dv, x, m, E(C)), 4 * n)
    add("anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", sh, (*d, dv, x, m, dm), 4 * n)
    add("anode_gpu_batch_mean_bwd_3d1_packed_f32", sh, (*d, dm, y), 4 * n)
    add("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", sh, (*d, dm, dx), 8 * n)
    # additive batch-norm entry points on the same arrays
    add("anode_gpu_batch_mean_var_3d1_packed_f32", sh, (*d, 1e-5, x, E(C), E(C)), 4 * n)
    add("anode_gpu_batch_mean_var_online_3d1_packed_f32", sh, (*d, 1e-5, 0.1, x, E(C), E(C), Rn(C), Rn(C)), 4 * n)
    add("anode_gpu_batch_norm_positive_clip_3d1_packed_f32", sh, (*d, x, m, v, y), 8 * n)
    add("anode_gpu_batch_norm_affine_3d1_packed_f32", sh, (*d, x, m, v, dm, dv, y), 8 * n)
    add("anode_gpu_batch_norm_bwd_reduce_3d1_packed_f32", sh, (*d, dy, x, m, v, None, E(C), E(C)), 8 * n)
    add("anode_gpu_batch_norm_bwd_apply_3d1_packed_f32", sh, (*d, dy, x, m, v, dm, dv, None, y), 12 * n)
    add("anode_gpu_bcast_flat_mult_add_I1b_I2abc_Oabc_packed_f32", sh, (*d, dm, x, dv, y), 8 * n)

    # flat maps and the join on the same 822 MB arrays
    fl = f"[{n}]"
    for name in ("copy", "modulus", "square", "sqrt", "positive_clip", "logistic", "unit_step", "normal_cdf", "tanh",
                 "rcosh2", "log_positive_clip", "positive_reciprocal"):
        add(f"anode_gpu_{name}_flat_map_f32", fl, (n, x, y), 8 * n)
    add("anode_gpu_leaky_relu_flat_map_f32", fl, (n, 0.1, x, y), 8 * n)
    add("anode_gpu_positive_clip_flat_map_bwd_f32", fl, (n, dy, x, y), 12 * n)
    add("anode_gpu_logistic_flat_map_bwd_f32", fl, (n, dy, x, y), 12 * n)
    add("anode_gpu_leaky_relu_flat_map_bwd_f32", fl, (n, 0.1, dy, x, y), 12 * n)
    add("anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32", fl, (n, dy, x, y), 12 * n)
    add("anode_gpu_add_packed_f32", fl, (n, x, dx), 12 * n)
    add("anode_gpu_set_constant_packed_f32", fl, (n, 0.0, y), 4 * n)
    add("anode_gpu_sum_packed_deterministic_f32", fl, (n, x, E(1)), 4 * n)

    # casts on [256,3,224,224]
    nq = 256 * 3 * 224 * 224
    q = torch.randint(0, 256, (nq,), device="cuda", dtype=torch.uint8, generator=g)
    add("anode_gpu_dequantize_u8_packed_f32", "[256,3,224,224]", (nq, 0.0, 1.0, q, y), 5 * nq)
    add("anode_gpu_upcast_u8_packed_u32", "[256,3,224,224]", (nq, q, E(nq, torch.int32)), 5 * nq)
    add("anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32", "[256,3,224,224]",
        (224 * 224, 3, 256, Rn(3), Rn(3), q, y), 5 * nq)
    add("anode_gpu_quantize_u8_packed_f32", "[256,3,224,224]", (nq, -4.0, 4.0, x, E(nq, torch.uint8)), 5 * nq)

    # row softmax / NLL: K = 10, 1000, 4096
    for K, R in ((10, 4 << 20), (1000, 65536), (4096, 16384)):
        lab = torch.randint(0, K, (R,), device="cuda", dtype=torch.int32, generator=g)
        rs = f"[{R},{K}]"
        add("anode_gpu_softmax_packed_block_f32", rs, (K, R, x, y), 8 * K * R)
        add("anode_gpu_softmax_packed_deterministic_f32", rs, (K, R, x, y), 8 * K * R)
        if K == 1000:
            add("anode_gpu_softmax_cat_nll_packed_f32", rs, (K, R, x, lab, E(R)), 12 * R)
            add("anode_gpu_softmax_cat_nll_bwd_packed_f32", rs, (K, R, dy, x, lab, y), 8 * K * R + 8 * R)
            add("anode_gpu_softmax_cat_nll_bwd_packed_accumulate_f32", rs, (K, R, dy, x, lab, dx), 12 * K * R + 8 * R)
            add("anode_gpu_arg_max_packed_u32", rs, (K, R, x, E(R, torch.int32)), 4 * K * R + 4 * R)
            add("anode_gpu_softmax_cat_nll_fused_packed_f32", rs, (K, R, x, lab, y, E(R)), 8 * K * R + 8 * R)
            add("anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32", rs, (K, R, x, lab, dy, y, E(R), dx),
                12 * K * R + 12 * R)

    # channel-axis softmax / NLL / one-hot / F1 on [8,19,512,1024]
    P, Cc, Nn = 512 * 1024, 19, 8
    ns = P * Cc * Nn
    lab = torch.randint(0, Cc, (P * Nn,), device="cuda", dtype=torch.int32, generator=g)
    ss = "[8,19,512,1024]"
    add("anode_gpu_softmax_nd_packed_f32", ss, (P, Cc, Nn, x, y), 8 * ns)
    add("anode_gpu_softmax_nd_cat_nll_packed_f32", ss, (P, Cc, Nn, x, lab, E(P * Nn)), 12 * P * Nn)
    add("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", ss, (P, Cc, Nn, dy, x, lab, y), 8 * ns + 8 * P * Nn)
    add("anode_gpu_softmax_nd_cat_nll_bwd_packed_accumulate_f32", ss, (P, Cc, Nn, dy, x, lab, dx), 12 * ns + 8 * P * Nn)
    add("anode_gpu_softmax_nd_cat_nll_fused_packed_f32", ss, (P, Cc, Nn, x, lab, y, E(P * Nn)), 8 * ns + 8 * P * Nn)
    add("anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32", ss, (P, Cc, Nn, x, lab, dy, y, E(P * Nn), dx),
        12 * ns + 12 * P * Nn)
    add("anode_gpu_discrete_one_hot_3d1_packed_f32", ss, (P, Cc, Nn, lab, y), 4 * P * Nn + 4 * ns)
    t01 = (torch.rand(ns, device="cuda", generator=g) < 0.3).float()
    add("anode_gpu_smooth_negative_f1_loss_3d1_packed_f32", ss, (P, Cc, Nn, 1e-3, x, t01, E(Cc * Nn)), 8 * ns)
    add("anode_gpu_smooth_negative_f1_loss_3d1_bwd_packed_f32", ss, (P, Cc, Nn, 1e-3, Rn(Cc * Nn), x, t01, y), 12 * ns)

    for sym, _, args, _ in L:
        gpu.call(sym, *args)
    torch.cuda.synchronize()
    times = [[] for _ in L]
    for _ in range(5):  # five runs of eleven rotations back to back, the first rotation of each run dropped (it starts on an idle GPU)
        runs = []
        for _ in range(11):
            evs = []
            for sym, _, args, _ in L:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                gpu.call(sym, *args)
                b.record()
                evs.append((a, b))
            runs.append(evs)
        torch.cuda.synchronize()
        for evs in runs[1:]:
            for i, (a, b) in enumerate(evs):
                times[i].append(a.elapsed_time(b) * 1e-3)
    assert gpu.take_last_error() == 0
    rows = []
    for (sym, shape, _, nbytes), ts in zip(L, times):
        t = sorted(ts)[len(ts) // 2]
        rows.append({"symbol": sym.replace("anode_gpu_", ""), "shape": shape, "us": round(t * 1e6, 1),
                     "min_us": round(min(ts) * 1e6, 1),
                     "gbps": round(nbytes / t / 1e9, 1), "pct_of_peak": round(100 * nbytes / t / 1e9 / HBM_PEAK_GBPS, 1)})
    return rows


def offset_views(torch, gpu):
    """Arrays that are views starting at any element (as_dptr() on a view): the entry points named below at the
    configs' shapes with every array on a 16-byte boundary, with every array one element past one (the same view of
    sibling arrays), and with the arrays 1, 2 and 3 elements past one (views that lie differently).  Launches of the
    three placements are made in rotation, back to back; median of 20."""
    E = lambda n, dt=torch.float32: torch.empty(n + 8, device="cuda", dtype=dt)  # noqa: E731
    placements = {"aligned": (0, 0, 0, 0), "all_plus_1": (1, 1, 1, 1), "plus_1_2_3": (1, 2, 3, 1)}
    cases = []

    def case(name, shape, nbytes, make):
        cases.append((name, shape, nbytes, make))

    def view(t, off, n):
        return t[off:off + n]

    for tag, (S, C, N) in (("cfg2a [256,64,112,112]", (12544, 64, 256)), ("cfg2b [256,2048,7,7]", (49, 2048, 256)),
                           ("cfg4 [2,32,128,128,128]", (128 ** 3, 32, 2))):
        n = S * C * N
        x, dy, y = torch.randn(n + 8, device="cuda"), torch.randn(n + 8, device="cuda"), E(n)
        m, v, dv, o = torch.randn(C + 8, device="cuda"), torch.rand(C + 8, device="cuda") + 0.5, torch.randn(C + 8, device="cuda"), E(C)
        d = (S, C, N)
        case("batch_mean_3d1_packed_f32", tag, 4 * n,
             lambda a, b, c, e, d=d, x=x, o=o, n=n, C=C: ("anode_gpu_batch_mean_3d1_packed_f32", (*d, view(x, a, n), view(o, e, C))))
        case("batch_norm_bwd_var_3d1_packed_f32", tag, 8 * n,
             lambda a, b, c, e, d=d, x=x, dy=dy, m=m, v=v, o=o, n=n, C=C:
             ("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", (*d, view(dy, a, n), view(x, b, n), view(m, e, C), view(v, e, C), view(o, e, C))))
        case("batch_norm_3d1_packed_f32", tag, 8 * n,
             lambda a, b, c, e, d=d, x=x, y=y, m=m, v=v, n=n, C=C:
             ("anode_gpu_batch_norm_3d1_packed_f32", (*d, view(x, a, n), view(m, e, C), view(v, e, C), view(y, b, n))))
        case("batch_var_bwd_3d1_packed_accumulate_f32", tag, 12 * n,
             lambda a, b, c, e, d=d, x=x, y=y, m=m, dv=dv, n=n, C=C:
             ("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", (*d, view(dv, e, C), view(x, a, n), view(m, e, C), view(y, b, n))))
        if tag.startswith("cfg4"):
            case("positive_clip_flat_map_f32", tag, 8 * n,
                 lambda a, b, c, e, x=x, y=y, n=n: ("anode_gpu_positive_clip_flat_map_f32", (n, view(x, a, n), view(y, b, n))))
            case("positive_clip_flat_map_bwd_f32", tag, 12 * n,
                 lambda a, b, c, e, x=x, y=y, dy=dy, n=n:
                 ("anode_gpu_positive_clip_flat_map_bwd_f32", (n, view(dy, a, n), view(x, b, n), view(y, c, n))))
    P, C, N = 512 * 1024, 19, 8
    n = P * C * N
    x, p, dx = torch.randn(n + 8, device="cuda"), E(n), E(n)
    lab = torch.randint(0, C, (P * N + 8,), device="cuda", dtype=torch.int32)
    dy, nll = torch.ones(P * N + 8, device="cuda"), E(P * N)
    tag = "cfg3b [8,19,512,1024]"
    case("softmax_nd_packed_f32", tag, 8 * n,
         lambda a, b, c, e: ("anode_gpu_softmax_nd_packed_f32", (P, C, N, view(x, a, n), view(p, b, n))))
    case("softmax_nd_cat_nll_bwd_packed_f32", tag, 8 * n + 8 * P * N,
         lambda a, b, c, e: ("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32",
                             (P, C, N, view(dy, e, P * N), view(p, a, n), view(lab, c, P * N), view(dx, b, n))))
    case("softmax_nd_cat_nll_fused_fwd_bwd_packed_f32", tag, 12 * n + 12 * P * N,
         lambda a, b, c, e: ("anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32",
                             (P, C, N, view(x, a, n), view(lab, c, P * N), view(dy, e, P * N), view(p, b, n),
                              view(nll, e, P * N), view(dx, c, n))))
    K, R = 1000, 65536
    case("softmax_packed_deterministic_f32", "[65536,1000]", 8 * K * R,
         lambda a, b, c, e: ("anode_gpu_softmax_packed_deterministic_f32", (K, R, view(x, a, K * R), view(p, b, K * R))))
    nq = 256 * 3 * 224 * 224
    q = torch.randint(0, 256, (nq + 32,), device="cuda", dtype=torch.uint8)
    zq = torch.empty(nq + 32, device="cuda", dtype=torch.uint8)
    tag = "cfg1 [256,3,224,224]"
    case("dequantize_u8_packed_f32", tag, 5 * nq,
         lambda a, b, c, e: ("anode_gpu_dequantize_u8_packed_f32", (nq, 0.0, 1.0, view(q, a, nq), view(p, b, nq))))
    case("quantize_u8_packed_f32", tag, 5 * nq,
         lambda a, b, c, e: ("anode_gpu_quantize_u8_packed_f32", (nq, -4.0, 4.0, view(x, a, nq), view(zq, b, nq))))

    rows = []
    for name, shape, nbytes, make in cases:
        calls = {k: make(*offs) for k, offs in placements.items()}
        for sym, args in calls.values():
            gpu.call(sym, *args)
        torch.cuda.synchronize()
        times = {k: [] for k in calls}
        rounds = []
        for _ in range(21):  # back to back; the first round, which starts on an idle GPU, is dropped
            evs = {}
            for k, (sym, args) in calls.items():
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                gpu.call(sym, *args)
                b.record()
                evs[k] = (a, b)
            rounds.append(evs)
        torch.cuda.synchronize()
        for evs in rounds[1:]:
            for k, (a, b) in evs.items():
                times[k].append(a.elapsed_time(b) * 1e-3)
        assert gpu.take_last_error() == 0
        row = {"symbol": name, "shape": shape}
        for k, ts in times.items():
            t = sorted(ts)[len(ts) // 2]
            row[k] = {"us": round(t * 1e6, 1), "gbps": round(nbytes / t / 1e9, 1)}
        row["all_plus_1_vs_aligned"] = round(row["all_plus_1"]["gbps"] / row["aligned"]["gbps"], 3)
        row["plus_1_2_3_vs_aligned"] = round(row["plus_1_2_3"]["gbps"] / row["aligned"]["gbps"], 3)
        rows.append(row)
    return rows


def graph_replay(torch, run_step, steps, step_bytes):
    """The same step captured once as a HIP graph and replayed: what the launch gaps cost (reported beside `value`,
    which stays the plainly launched figure)."""
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        run_step()  # the reductions' scratch for this stream exists before capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        run_step()
    graph.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        graph.replay()
    torch.cuda.synchronize()
    g_s = (time.perf_counter() - t0) / steps
    return {"ms_per_step": round(g_s * 1e3, 4), "gbps": round(step_bytes / g_s / 1e9, 1),
            "pct_of_hbm_peak": round(100 * step_bytes / g_s / 1e9 / HBM_PEAK_GBPS, 2)}


def small_shape_latency(torch, gpu, groups, passes=100):
    """Launch-bound shapes (config 0, config 3a): time per pass over `passes` back-to-back passes, launched one entry
    point at a time and as one captured HIP graph replayed.  Separates launch latency from bandwidth."""
    out = {}
    stream = torch.cuda.Stream()
    for name, ls in groups.items():
        def run():
            for l in ls:
                gpu.call(l.symbol, *l.args)
        with torch.cuda.stream(stream):
            run()  # allocates the reductions' scratch for this stream before anything is captured
            run()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            run()
        times = {}
        for kind, once in (("eager", run), ("graph", graph.replay)):
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            with torch.cuda.stream(stream):
                once()
                a.record()
                for _ in range(passes):
                    once()
                b.record()
            stream.synchronize()
            times[kind] = a.elapsed_time(b) * 1e-3 / passes
        nbytes = sum(l.alg_bytes for l in ls)
        out[name] = {"launches": len(ls), "eager_us_per_pass": round(times["eager"] * 1e6, 2),
                     "graph_us_per_pass": round(times["graph"] * 1e6, 2),
                     "graph_gbps": round(nbytes / times["graph"] / 1e9, 1)}
    return out


def small_shape_groups(torch, launches, fused=()):
    """Config 0 (BN on [32,16,28,28], softmax + NLL on [32,10]) and the config 3a launches of the step."""
    def empty(n):
        return torch.empty(n, device="cuda")
    S, C, N = 784, 16, 32
    n = S * C * N
    x, dy, y, dx = torch.randn(n, device="cuda"), torch.randn(n, device="cuda"), empty(n), empty(n)
    m, v, dm, dv = empty(C), empty(C), empty(C), empty(C)
    d = (S, C, N)
    bn0 = [Launch("bn_cfg0", "anode_gpu_batch_mean_3d1_packed_f32", (*d, x, m), 4 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_var_3d1_packed_f32", (*d, 1e-5, x, m, v), 4 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_norm_3d1_packed_f32", (*d, x, m, v, y), 8 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_norm_bwd_3d1_packed_f32", (*d, dy, v, dx), 8 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", (*d, dy, v, dm), 4 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_norm_bwd_var_3d1_packed_f32", (*d, dy, x, m, v, dv), 8 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", (*d, dv, x, m, dx), 12 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", (*d, dv, x, m, dm), 4 * n, n),
           Launch("bn_cfg0", "anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", (*d, dm, dx), 8 * n, n)]
    K, R = 10, 32
    lg, p, nll, dl = torch.randn(K * R, device="cuda"), empty(K * R), empty(R), empty(K * R)
    lab = torch.randint(0, K, (R,), device="cuda", dtype=torch.int32)
    ones = torch.ones(R, device="cuda")
    sm0 = [Launch("softmax_cfg0", "anode_gpu_softmax_packed_block_f32", (K, R, lg, p), 8 * K * R, K * R),
           Launch("softmax_cfg0", "anode_gpu_softmax_cat_nll_packed_f32", (K, R, p, lab, nll), 12 * R, R),
           Launch("softmax_cfg0", "anode_gpu_softmax_cat_nll_bwd_packed_f32", (K, R, ones, p, lab, dl), 8 * K * R + 8 * R, K * R)]
    groups = {"bn_fwd_bwd_cfg0": bn0, "softmax_nll_cfg0": sm0}
    cfg3a = [l for l in launches if l.group == "softmax_cfg3a"]
    if cfg3a:
        groups["softmax_nll_cfg3a"] = cfg3a
    cfg3a_fused = [l for l in fused if l.group == "fused_softmax_cfg3a"]
    if cfg3a_fused:
        groups["softmax_nll_cfg3a_fused_fwd"] = cfg3a_fused  # softmax + NLL in one launch, then the backward
    one = [l for l in fused if l.group == "fused_softmax_fwd_bwd_cfg3a"]
    if one:
        groups["softmax_nll_cfg3a_one_launch"] = one         # softmax + NLL + backward in one launch
    return groups


def cpu_baseline():
    """The fp32 CPU restatement (reference operation order) on a bounded sample of the same workload."""
    import numpy as np

    from oracle import binding as o

    host_cpus = os.cpu_count() or 1
    omp_default = o.max_threads()
    threads = min(16, host_cpus)  # the GPU box grants 16 cores per GPU whatever nproc shows
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

    # inputs: a 64-sample slice of config 2a, four samples of config 3b, all 256 images of config 1
    S, C, N = 112 * 112, 64, 64
    d = (S, C, N)
    n_bn = S * C * N
    x = (2 + 3 * g.standard_normal(n_bn, dtype=np.float32)).astype(F32)
    dy = g.standard_normal(n_bn, dtype=np.float32)
    P, K, M = 512 * 1024, 19, 4
    n_sm = P * K * M
    logits = g.standard_normal(n_sm, dtype=np.float32)
    lab = g.integers(0, K, P * M).astype(np.uint32)
    ones = np.ones(P * M, F32)
    n_q = 256 * 3 * 224 * 224
    q = g.integers(0, 256, n_q, dtype=np.uint8)
    st = {}

    def one_pass():
        n = n_bn
        timed("bn", 4 * n, lambda: st.__setitem__("m", o.batch_mean(*d, x)))
        timed("bn", 4 * n, lambda: st.__setitem__("v", o.batch_var(*d, 1e-5, x, st["m"])))
        timed("bn", 8 * n, lambda: o.batch_norm(*d, x, st["m"], st["v"]))
        timed("bn", 8 * n, lambda: st.__setitem__("dx", o.batch_norm_bwd(*d, dy, st["v"])))
        timed("bn", 4 * n, lambda: st.__setitem__("dm", o.batch_norm_bwd_mean(*d, dy, st["v"])))
        timed("bn", 8 * n, lambda: st.__setitem__("dv", o.batch_norm_bwd_var(*d, dy, x, st["m"], st["v"])))
        timed("bn", 12 * n, lambda: st.__setitem__("dx", o.batch_var_bwd(*d, st["dv"], x, st["m"], dx_in=st["dx"])))
        timed("bn", 4 * n, lambda: st.__setitem__("dm", o.batch_var_bwd_mean(*d, st["dv"], x, st["m"], dmean_in=st["dm"])))
        timed("bn", 8 * n, lambda: o.batch_mean_bwd(*d, st["dm"], dx_in=st["dx"]))
        n = n_sm
        timed("softmax_nll", 8 * n, lambda: st.__setitem__("p", o.softmax_nd(P, K, M, logits)))
        timed("softmax_nll", 12 * P * M, lambda: o.softmax_nd_cat_nll(P, K, M, st["p"], lab))
        timed("softmax_nll", 8 * n + 8 * P * M, lambda: o.softmax_nd_cat_nll_bwd(P, K, M, ones, st["p"], lab))
        timed("cast", 5 * n_q, lambda: o.dequantize_u8(0.0, 1.0, q))
        timed("cast", 5 * n_q, lambda: o.upcast_u8(q))

    # BASELINE config 0, the configuration named as the CPU reference path: BN fwd+bwd on [32,16,28,28] (the nine
    # reference launches) and softmax + NLL + backward on [32,10], per pass, on one thread and on all cores
    def config0(nthreads):
        o.set_threads(nthreads)
        S0, C0, N0 = 784, 16, 32
        d0 = (S0, C0, N0)
        g0 = np.random.default_rng(0)
        x0 = g0.standard_normal(S0 * C0 * N0).astype(F32)
        dy0 = g0.standard_normal(S0 * C0 * N0).astype(F32)
        lg0 = g0.standard_normal(320).astype(F32)
        lab0 = g0.integers(0, 10, 32).astype(np.uint32)
        one0 = np.ones(32, F32)

        def bn():
            m = o.batch_mean(*d0, x0)
            v = o.batch_var(*d0, 1e-5, x0, m)
            o.batch_norm(*d0, x0, m, v)
            dx = o.batch_norm_bwd(*d0, dy0, v)
            dm = o.batch_norm_bwd_mean(*d0, dy0, v)
            dv = o.batch_norm_bwd_var(*d0, dy0, x0, m, v)
            dx = o.batch_var_bwd(*d0, dv, x0, m, dx_in=dx)
            dm = o.batch_var_bwd_mean(*d0, dv, x0, m, dmean_in=dm)
            o.batch_mean_bwd(*d0, dm, dx_in=dx)

        def sm():
            pr = o.softmax(10, 32, lg0)
            o.softmax_cat_nll(10, 32, pr, lab0)
            o.softmax_cat_nll_bwd(10, 32, one0, pr, lab0)

        res = {}
        for name, fn, reps in (("bn_fwd_bwd_cfg0", bn, 40), ("softmax_nll_cfg0", sm, 400)):
            fn()
            t0 = time.perf_counter()
            for _ in range(reps):
                fn()
            res[name] = round((time.perf_counter() - t0) / reps * 1e6, 1)
        return res

    cfg0_one, cfg0_all = config0(1), config0(threads)
    o.set_threads(threads)

    # repeat the sample until about 1.5 s of wall time on `threads` cores (~20-30 core-seconds), at most 16 passes
    passes = 0
    while passes < 16 and (passes == 0 or total_s < 1.5):
        one_pass()
        passes += 1
    multi = (total_bytes, total_s, dict(parts), passes)
    # the same sample once on one thread (the scalar figure beside the threaded one)
    o.set_threads(1)
    total_bytes, total_s = 0, 0.0
    parts.clear()
    one_pass()
    single_gbps = total_bytes / total_s / 1e9
    single_s = total_s
    o.set_threads(threads)
    total_bytes, total_s, parts, passes = multi
    return {
        "value": round(total_bytes / total_s / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "host_cpus_reported": host_cpus,
        "omp_max_threads_default": omp_default,
        "single_thread": {"value": round(single_gbps, 3), "unit": "GB/s", "cores": 1, "seconds": round(single_s, 2)},
        "kind": "port",
        "sample": "fp32 CPU restatement, OpenMP: BN fwd+bwd (9 launches) on [64,64,112,112]; softmax_nd+NLL+bwd on "
                  "[4,19,512,1024]; dequantize+upcast on [256,3,224,224]; repeated to ~1.5 s; algorithmic bytes / time",
        "parts_gbps": {k: round(b / s / 1e9, 3) for k, (b, s) in parts.items()},
        "seconds": round(total_s, 2),
        "passes": passes,
        "config0_us_per_pass": {k: {"cpu_us_1_thread": cfg0_one[k], f"cpu_us_{threads}_threads": cfg0_all[k]} for k in cfg0_one},
        "config0_note": "BASELINE configs[0] (BN fwd+bwd [32,16,28,28], nine launches; softmax + NLL + backward [32,10], "
                        "three launches) through the same fp32 restatement, called from Python (each call carries a few "
                        "microseconds of ctypes overhead); the GPU figures for the same launches are small_shapes.*",
    }


def main():
    args = parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        sys.stderr.write("bench.py: this build measures one GPU; --gpus above 1 is not supported\n")
        sys.exit(2)
    if args.source_fingerprints:
        print(json.dumps(source_fingerprints()), flush=True)
        return
    import torch

    from anode_amd import gpu

    if not torch.cuda.is_available():
        sys.stderr.write("bench.py: no GPU visible\n")
        sys.exit(3)
    torch.cuda.set_device(0)
    if args.stream_probe:
        print(json.dumps({"stream_probe": stream_probe(torch, gpu)}), flush=True)
        return
    if args.shape_sweep:
        print(json.dumps({"shape_sweep": shape_sweep(torch, gpu), "peak_gbps": HBM_PEAK_GBPS}), flush=True)
        return
    if args.all_symbols:
        print(json.dumps({"all_symbols": all_symbols(torch, gpu), "peak_gbps": HBM_PEAK_GBPS}), flush=True)
        return
    if args.offset_views:
        print(json.dumps({"offset_views": offset_views(torch, gpu), "peak_gbps": HBM_PEAK_GBPS}), flush=True)
        return
    only = set(filter(None, args.only.split(",")))
    launches, fused = build_workload(torch, only, args.copy_calibration)
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
    # (11 passes back to back, the first dropped: a launch made on an idle GPU, as the first launch after a
    # synchronisation is, measures about 6 us more between its events than the same launch inside a sequence)
    per_launch = [[] for _ in launches]
    all_evs = []
    for _ in range(11):
        evs = []
        for l in launches:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            gpu.call(l.symbol, *l.args)
            b.record()
            evs.append((a, b))
        all_evs.append(evs)
    torch.cuda.synchronize()
    for evs in all_evs[1:]:
        for i, (a, b) in enumerate(evs):
            per_launch[i].append(a.elapsed_time(b) * 1e-3)
    med = [sorted(t)[len(t) // 2] for t in per_launch]
    dom_i = max(range(len(launches)), key=lambda i: med[i])
    dom = launches[dom_i]

    # the same step with one event pair per composite (a config's launch set, in step order): what a caller of the
    # whole composite sees, including the gaps between its launches but without an event pair around each of them
    order = []
    for l in launches:
        if not order or order[-1] != l.group:
            order.append(l.group)
    per_group = {k: [] for k in order}
    passes = []
    for _ in range(11):  # back to back, no synchronisation in between: the first pass (which starts on an idle GPU) is dropped
        marks, prev = [], None
        for l in launches:
            if l.group != prev:
                e = torch.cuda.Event(enable_timing=True)
                e.record()
                marks.append(e)
                prev = l.group
            gpu.call(l.symbol, *l.args)
        e = torch.cuda.Event(enable_timing=True)
        e.record()
        marks.append(e)
        passes.append(marks)
    torch.cuda.synchronize()
    for marks in passes[1:]:
        for i, k in enumerate(order):
            per_group[k].append(marks[i].elapsed_time(marks[i + 1]) * 1e-3)
    group_med = {k: sorted(t)[len(t) // 2] for k, t in per_group.items()}

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
        "traffic_source": TRAFFIC_SOURCE,
    }
    fingerprints = source_fingerprints()
    roofline["traffic"], note = measured_traffic(dom.symbol, dom.group, fingerprints)
    if note:
        roofline["traffic_note"] = note
        sys.stderr.write(f"bench.py: roofline.traffic: {note}\n")
    # the same counters for the dominant kernel of every config (bytes per launch; ratio to the algorithmic bytes)
    traffic_by_kernel = []
    for l in launches:
        t, note = measured_traffic(l.symbol, l.group, fingerprints)
        if t is not None:
            traffic_by_kernel.append({"group": l.group, "symbol": l.symbol.replace("anode_gpu_", ""),
                                      "alg_bytes": l.alg_bytes, "traffic": t, "ratio": round(t / l.alg_bytes, 3)})
        elif note:
            traffic_by_kernel.append({"group": l.group, "symbol": l.symbol.replace("anode_gpu_", ""),
                                      "alg_bytes": l.alg_bytes, "traffic": None, "note": note})

    groups = {}
    for l, t in zip(launches, med):
        b, s, e = groups.get(l.group, (0, 0.0, 0))
        groups[l.group] = (b + l.alg_bytes, s + t, e + l.elements)
    # per composite: time between the events at its two ends; `sum_of_launches_us` is the sum of its launches timed
    # one by one (per_symbol), which carries one event pair per launch
    groups = {k: (b, group_med[k], e, s) for k, (b, s, e) in groups.items()}
    breakdown = {k: {"gbps": round(b / s / 1e9, 1), "pct_of_peak": round(100 * b / s / 1e9 / HBM_PEAK_GBPS, 1),
                     "us": round(s * 1e6, 1), "gelem_per_s": round(e / s / 1e9, 2),
                     "sum_of_launches_us": round(s1 * 1e6, 1)} for k, (b, s, e, s1) in groups.items()}
    per_symbol = [{"group": l.group, "symbol": l.symbol.replace("anode_gpu_", ""), "us": round(t * 1e6, 1),
                   "min_us": round(min(ts) * 1e6, 1), "gbps": round(l.alg_bytes / t / 1e9, 1)}
                  for l, t, ts in zip(launches, med, per_launch)]

    # the additive (fused) entry points on the same data: time per group over the fused byte model, and the
    # time of the reference-ABI launches that do the same work
    fused_model = {}
    if fused:
        for l in fused:
            gpu.call(l.symbol, *l.args)
        torch.cuda.synchronize()
        ftimes = [[] for _ in fused]
        all_evs = []
        for _ in range(11):  # back to back, the first pass dropped (see above)
            evs = []
            for l in fused:
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record()
                gpu.call(l.symbol, *l.args)
                b.record()
                evs.append((a, b))
            all_evs.append(evs)
        torch.cuda.synchronize()
        for evs in all_evs[1:]:
            for i, (a, b) in enumerate(evs):
                ftimes[i].append(a.elapsed_time(b) * 1e-3)
        assert gpu.take_last_error() == 0
        forder = []
        for l in fused:
            if not forder or forder[-1] != l.group:
                forder.append(l.group)
        fgroup = {k: [] for k in forder}
        fpasses = []
        for _ in range(11):
            marks, prev = [], None
            for l in fused:
                if l.group != prev:
                    e = torch.cuda.Event(enable_timing=True)
                    e.record()
                    marks.append(e)
                    prev = l.group
                gpu.call(l.symbol, *l.args)
            e = torch.cuda.Event(enable_timing=True)
            e.record()
            marks.append(e)
            fpasses.append(marks)
        torch.cuda.synchronize()
        for marks in fpasses[1:]:
            for i, k in enumerate(forder):
                fgroup[k].append(marks[i].elapsed_time(marks[i + 1]) * 1e-3)
        fg = {}
        for l in fused:
            b, s_ = fg.get(l.group, (0, 0.0))
            fg[l.group] = (b + l.alg_bytes, sorted(fgroup[l.group])[len(fgroup[l.group]) // 2])
        abi_time = {k: v[1] for k, v in groups.items()}
        same_work = {
            "fused_bn_fwd_cfg2a": ["bn_fwd_cfg2a"], "fused_bn_bwd_cfg2a": ["bn_bwd_cfg2a"],
            "fused_bn_fwd_cfg2b": ["bn_fwd_cfg2b"], "fused_bn_bwd_cfg2b": ["bn_bwd_cfg2b"],
            "fused_bn_fwd_cfg4": ["bn_fwd_cfg4", "relu_cfg4:positive_clip_flat_map_f32"],
            "fused_bn_bwd_cfg4": ["bn_bwd_cfg4", "relu_cfg4:positive_clip_flat_map_bwd_f32"],
            "fused_softmax_fwd_cfg3b": ["softmax_cfg3b:softmax_nd_packed_f32", "softmax_cfg3b:softmax_nd_cat_nll_packed_f32"],
            "fused_softmax_fwd_bwd_cfg3b": ["softmax_cfg3b"],
            "fused_softmax_cfg3a": ["softmax_cfg3a"],
            "fused_softmax_fwd_bwd_cfg3a": ["softmax_cfg3a"],
        }
        sym_time = {f"{l.group}:{l.symbol.replace('anode_gpu_', '')}": t for l, t in zip(launches, med)}
        for k, (b, s_) in fg.items():
            entry = {"gbps": round(b / s_ / 1e9, 1), "pct_of_peak": round(100 * b / s_ / 1e9 / HBM_PEAK_GBPS, 1),
                     "us": round(s_ * 1e6, 1)}
            parts = same_work.get(k)
            if parts and all((p_ in abi_time) or (p_ in sym_time) for p_ in parts):
                abi_s = sum(abi_time[p_] if p_ in abi_time else sym_time[p_] for p_ in parts)
                entry["abi_sequence_us"] = round(abi_s * 1e6, 1)
                entry["speedup_vs_abi_sequence"] = round(abi_s / s_, 2)
            entry["launches"] = [{"symbol": l.symbol.replace("anode_gpu_", ""), "us": round(sorted(t)[len(t) // 2] * 1e6, 1)}
                                 for l, t in zip(fused, ftimes) if l.group == k]
            fused_model[k] = entry
        if "fused_cast_cfg1" in fused_model:
            fused_model["fused_cast_cfg1"]["note"] = ("what config 1 names beyond the reference's casts: u8 -> f32 with "
                                                      "per-channel normalisation in one pass, then f32 -> u8 quantisation; "
                                                      "quantize is parity unpinned by the reference (it has no such kernel)")
        for k in ("affine_bn_fwd_cfg2a", "affine_bn_fwd_cfg2b"):
            if k in fused_model:
                fused_model[k]["note"] = ("config 2's gamma ~ U(0.5,1.5), beta ~ N(0,0.1), momentum 0.1: single-pass "
                                          "statistics, normalise + affine, online_average of mean and var (C elements each)")
        for k in ("affine_one_stats_launch_bn_fwd_cfg2a", "affine_one_stats_launch_bn_fwd_cfg2b"):
            if k in fused_model:
                fused_model[k]["note"] = ("the same layer in two launches: the statistics launch also moves the running "
                                          "mean and variance (bit-identical to the four launches of affine_bn_fwd_*)")

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
        "data": "synthetic: numpy.random.default_rng(0), drawn in float64 and cast to float32, labels from integers()",
        "config": {
            "workload": "configs[1..4], ABI byte model: cast+dequantize u8[256,3,224,224]; BN fwd(3)+bwd(6 launches) "
                        "f32 [256,64,112,112], [256,2048,7,7], [2,32,128,128,128] + ReLU fwd/bwd; softmax+NLL+bwd "
                        "[256,1000] and [8,19,512,1024]",
            "launches_per_step": len(launches),
            "alg_bytes_per_step": step_bytes,
            "inputs": "one generator, in this order: cfg1 codes integers(0,256), N(0,1) tensor to quantise; cfg2a then "
                      "cfg2b x = 2 + 3 N(0,1), dy = N(0,1), gamma = U(0.5,1.5), beta = N(0,0.1); cfg3a logits = 2 N(0,1) "
                      "(variance 4), labels integers(0,1000); cfg3b logits N(0,1), labels integers(0,19) with "
                      "random() < 0.05 set to 255, dy = 1; cfg4 x = N(0,1), dy = N(0,1), gamma = 1, beta = 0; eps 1e-5",
        },
        "pct_of_hbm_peak": round(100 * value / HBM_PEAK_GBPS, 2),
        "gelem_per_s": round(step_elems / step_s / 1e9, 2),
        "roofline": roofline,
        "traffic_by_kernel": traffic_by_kernel,
        "breakdown": breakdown,
        "fused_model": fused_model,
        "per_symbol": per_symbol,
    }
    if not only:
        # side measurements: a failure in one of them is recorded and must not cost the headline line
        try:
            out["graph_replay"] = graph_replay(torch, run_step, args.steps, step_bytes)
        except Exception as e:  # noqa: BLE001
            out["graph_replay"] = {"error": repr(e)}
        try:
            out["small_shapes"] = small_shape_latency(torch, gpu, small_shape_groups(torch, launches, fused))
        except Exception as e:  # noqa: BLE001
            out["small_shapes"] = {"error": repr(e)}
    if not args.no_cpu_baseline:
        try:
            out["cpu_baseline"] = cpu_baseline()
        except Exception as e:  # noqa: BLE001
            out["cpu_baseline"] = {"error": repr(e)}
    cb = out.get("cpu_baseline", {})
    if isinstance(out.get("small_shapes"), dict) and "config0_us_per_pass" in cb:
        for k, v in cb["config0_us_per_pass"].items():
            if k in out["small_shapes"]:
                out["small_shapes"][k]["cpu_us"] = v
    out["targets"] = targets_block(breakdown, fused_model)
    print(json.dumps(out), flush=True)


def targets_block(breakdown, fused_model):
    """north_star's bar, machine-readable: every composite with its byte model and whether it sustains 70 % of the
    8 TB/s HBM peak.  Launch-bound composites (config 3a: 1 MB arrays) are listed and flagged as such."""
    notes = {
        "softmax_cfg3a": "launch-bound: 1 MB arrays, 0.26 us at peak",
        "fused_softmax_cfg3a": "launch-bound: 1 MB arrays",
        "fused_softmax_fwd_bwd_cfg3a": "launch-bound: 1 MB arrays",
        "softmax_cfg3b": "the reference ABI splits softmax and the label gather: with uniformly random labels the gather "
                         "must touch 86 % of the probability tensor's 128-byte lines for 4 bytes per pixel (5.8 x its "
                         "byte model), which holds this composite under 70 %; fused_softmax_fwd_cfg3b and "
                         "fused_softmax_fwd_bwd_cfg3b are the same work without the gather",
    }
    out = {}
    for model, table in (("abi", breakdown), ("fused", fused_model)):
        for k, v in table.items():
            e = {"pct_of_peak": v["pct_of_peak"], "byte_model": model, "met_70": bool(v["pct_of_peak"] >= 70.0)}
            if k in notes:
                e["note"] = notes[k]
            out[k] = e
    return out


if __name__ == "__main__":
    main()
