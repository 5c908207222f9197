"""GPU parity on seeded random shapes and pointer alignments, with guard bands.

The shape lists of the other parity tests are chosen by hand to reach each
tiling and access width; this file draws shapes and element offsets from a
fixed generator instead, so that combinations nobody thought of are covered
too.  Every output lies between two guard bands that must come back untouched:
a store that strays outside its array fails here even where it lands in memory
the process owns.
"""
import os

import numpy as np
import pytest
import torch

from gpu_util import F32, assert_bit_exact, assert_close, call, dev, host, rms

pytestmark = pytest.mark.gpu

GUARD = 64  # elements on either side of an output
SCALE = max(1, int(os.environ.get("ANODE_DRAWN_CASES_SCALE", "1")))  # a longer campaign on demand
BUDGET = int(os.environ.get("ANODE_DRAWN_ELEMENTS", str(1 << 20)))      # most elements of a drawn array


class Guarded:
    """An output array of n elements at `offset` elements past a 256-byte boundary, between two bands of a
    sentinel value."""

    def __init__(self, n, offset=0, dtype=torch.float32, init=None):
        self.n = n
        self.dtype = dtype
        self.sentinel = 77 if dtype in (torch.uint8, torch.int32) else -12345.0
        self.buf = torch.full((GUARD + offset + n + GUARD,), self.sentinel, dtype=dtype, device="cuda")
        self.view = self.buf[GUARD + offset:GUARD + offset + n]
        self.lo = GUARD + offset
        if init is not None:
            self.view.copy_(torch.from_numpy(np.ascontiguousarray(init).ravel()))
        elif dtype == torch.float32:
            self.view.fill_(float("nan"))

    def get(self, what):
        torch.cuda.synchronize()
        whole = self.buf.cpu().numpy()
        assert np.all(whole[:self.lo] == self.sentinel), f"{what}: wrote below the array"
        assert np.all(whole[self.lo + self.n:] == self.sentinel), f"{what}: wrote past the array"
        return whole[self.lo:self.lo + self.n]


def log_uniform(g, lo, hi):
    return int(round(float(np.exp(g.uniform(np.log(lo), np.log(hi + 1))))) // 1) or lo


def draw_scn(g, budget=BUDGET):
    """(S, C, N) with S*C*N <= budget; S, C, N spread over orders of magnitude."""
    while True:
        S = min(log_uniform(g, 1, 9000 * (BUDGET >> 20)), 9000 * (BUDGET >> 20))
        C = min(log_uniform(g, 1, 700), 700)
        N = min(log_uniform(g, 1, 70), 70)
        if S * C * N <= budget:
            return S, C, N


BN_CASES = [draw_scn(np.random.default_rng(1000 + i)) + (int(np.random.default_rng(200000 + i).integers(0, 4)),)
            for i in range(28 * SCALE)]


@pytest.mark.parametrize("S,C,N,offset", BN_CASES)
def test_batch_norm_family_on_drawn_shapes(oracle, S, C, N, offset):
    print(f"case S={S} C={C} N={N} offset={offset}", flush=True)
    g = np.random.default_rng(S * 7 + C * 3 + N)
    n = S * C * N
    dims = (S, C, N)
    eps = 1e-5
    x = (1.5 + 2.0 * g.standard_normal(n)).astype(F32)
    dy = g.standard_normal(n).astype(F32)
    old = g.standard_normal(n).astype(F32)
    oldc = g.standard_normal(C).astype(F32)
    xd, dyd = dev(x, offset), dev(dy, offset)

    mean_o = Guarded(C, offset)
    call("anode_gpu_batch_mean_3d1_packed_f32", *dims, xd, mean_o.view)
    mean = mean_o.get("mean")
    assert_close(mean, oracle.batch_mean(*dims, x, f64=True), "mean")

    var_o = Guarded(C, offset)
    call("anode_gpu_batch_var_3d1_packed_f32", *dims, eps, xd, mean_o.view, var_o.view)
    var = var_o.get("var")
    assert_close(var, oracle.batch_var(*dims, eps, x, mean, f64=True), "var")

    # single-pass statistics agree with the two launches
    m2, v2 = Guarded(C, offset), Guarded(C, offset)
    call("anode_gpu_batch_mean_var_3d1_packed_f32", *dims, eps, xd, m2.view, v2.view)
    assert_close(m2.get("mean_var mean"), oracle.batch_mean(*dims, x, f64=True), "single-pass mean")
    assert_close(v2.get("mean_var var"), oracle.batch_var(*dims, eps, x, mean, f64=True), "single-pass var",
                 abs_floor=1e-6)

    y_o = Guarded(n, offset)
    call("anode_gpu_batch_norm_3d1_packed_f32", *dims, xd, mean_o.view, var_o.view, y_o.view)
    assert_bit_exact(y_o.get("norm"), oracle.batch_norm(*dims, x, mean, var), "norm")

    out = Guarded(C, offset, init=oldc)
    call("anode_gpu_batch_norm_bwd_var_3d1_packed_accumulate_f32", *dims, dyd, xd, mean_o.view, var_o.view, out.view)
    ref = oracle.batch_norm_bwd_var(*dims, dy, x, mean, var, dvar_in=oldc, f64=True)
    assert_close(out.get("norm_bwd_var"), ref, "norm_bwd_var_accumulate", abs_floor=1e-6 * rms(ref))

    out = Guarded(C, offset)
    call("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", *dims, dyd, var_o.view, out.view)
    ref = oracle.batch_norm_bwd_mean(*dims, dy, var, f64=True)
    assert_close(out.get("norm_bwd_mean"), ref, "norm_bwd_mean", abs_floor=1e-6 * rms(ref))

    dvar = g.standard_normal(C).astype(F32)
    out = Guarded(n, offset, init=old)
    call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *dims, dev(dvar), xd, mean_o.view, out.view)
    assert_bit_exact(out.get("var_bwd"), oracle.batch_var_bwd(*dims, dvar, x, mean, dx_in=old), "var_bwd_accumulate")

    out = Guarded(n, offset)
    call("anode_gpu_batch_norm_bwd_3d1_packed_f32", *dims, dyd, var_o.view, out.view)
    assert_bit_exact(out.get("norm_bwd"), oracle.batch_norm_bwd(*dims, dy, var), "norm_bwd")


CAST_CASES = []
for i in range(24 * SCALE):
    _g = np.random.default_rng(3000 + i)
    CAST_CASES.append((log_uniform(_g, 1, 60000), log_uniform(_g, 1, 5), log_uniform(_g, 1, 6),
                       int(_g.integers(0, 16)), int(_g.integers(0, 4))))


@pytest.mark.parametrize("S,C,N,off_u8,off_f32", CAST_CASES)
def test_casts_on_drawn_shapes(oracle, S, C, N, off_u8, off_f32):
    print(f"case S={S} C={C} N={N} off_u8={off_u8} off_f32={off_f32}", flush=True)
    g = np.random.default_rng(S + 11 * C + N)
    n = S * C * N
    q = g.integers(0, 256, n).astype(np.uint8)
    qd = dev(q, off_u8)

    out = Guarded(n, off_f32, dtype=torch.int32)
    call("anode_gpu_upcast_u8_packed_u32", n, qd, out.view)
    assert np.array_equal(out.get("upcast").astype(np.uint32), q.astype(np.uint32))

    out = Guarded(n, off_f32)
    call("anode_gpu_dequantize_u8_packed_f32", n, -1.0, 2.5, qd, out.view)
    assert_bit_exact(out.get("dequantize"), oracle.dequantize_u8(-1.0, 2.5, q), "dequantize")

    a = g.uniform(0.5, 1.5, C).astype(F32)
    b = g.standard_normal(C).astype(F32)
    out = Guarded(n, off_f32)
    call("anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32", S, C, N, dev(a), dev(b), qd, out.view)
    assert_bit_exact(out.get("bcast dequantize"), oracle.bcast_dequantize_u8(S, C, N, a, b, q), "bcast dequantize")

    x = g.uniform(-1.5, 3.0, n).astype(F32)
    out = Guarded(n, off_u8, dtype=torch.uint8)
    call("anode_gpu_quantize_u8_packed_f32", n, -1.0, 2.5, dev(x, off_f32), out.view)
    assert np.array_equal(out.get("quantize"), oracle.quantize_u8(-1.0, 2.5, x))


ROW_CASES = []
for i in range(24 * SCALE):
    _g = np.random.default_rng(40000 + i)
    K = log_uniform(_g, 1, 200000)
    ROW_CASES.append((K, max(1, min(log_uniform(_g, 1, 3000), (BUDGET >> 1) // K)), int(_g.integers(0, 4))))


@pytest.mark.parametrize("K,R,offset", ROW_CASES)
def test_row_softmax_head_on_drawn_shapes(oracle, K, R, offset):
    print(f"case K={K} R={R} offset={offset}", flush=True)
    g = np.random.default_rng(K * 5 + R)
    x = (2.0 * g.standard_normal(K * R)).astype(F32)
    lab = g.integers(0, K, R).astype(np.uint32)
    dy = g.standard_normal(R).astype(F32)
    xd, labd, dyd = dev(x, offset), dev(lab.view(np.int32), offset), dev(dy, offset)
    cfg_block = 1024

    p_o = Guarded(K * R, offset)
    name = "anode_gpu_softmax_packed_block_f32" if K <= cfg_block else "anode_gpu_softmax_packed_deterministic_f32"
    call(name, K, R, xd, p_o.view)
    p = p_o.get("softmax")
    ref = oracle.softmax(K, R, x, f64=True)
    assert_close(p, ref, "softmax", abs_floor=1e-30)

    nll_o = Guarded(R, offset)
    call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p_o.view, labd, nll_o.view)
    nll = nll_o.get("nll")
    assert_close(nll, oracle.softmax_cat_nll(K, R, p, lab, f64=True), "nll", abs_floor=1e-6)

    dx_o = Guarded(K * R, offset)
    call("anode_gpu_softmax_cat_nll_bwd_packed_f32", K, R, dyd, p_o.view, labd, dx_o.view)
    dx = dx_o.get("nll bwd")
    assert_bit_exact(dx, oracle.softmax_cat_nll_bwd(K, R, dy, p, lab), "nll bwd")

    # the one-launch forms give the same bits as the launches above
    p2, n2, d2 = Guarded(K * R, offset), Guarded(R, offset), Guarded(K * R, offset)
    call("anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32", K, R, xd, labd, dyd, p2.view, n2.view, d2.view)
    assert_bit_exact(p2.get("fused softmax"), p, "fused softmax")
    assert_bit_exact(n2.get("fused nll"), nll, "fused nll")
    assert_bit_exact(d2.get("fused dx"), dx, "fused dx")


ND_CASES = []
for i in range(20 * SCALE):
    _g = np.random.default_rng(500000 + i)
    C = log_uniform(_g, 1, 700)
    ND_CASES.append((max(1, min(log_uniform(_g, 1, 40000), (BUDGET >> 1) // C)), C, log_uniform(_g, 1, 4),
                     int(_g.integers(0, 4))))
# short planes of whole 16-byte groups with more than 32 classes: the kernels that keep whole samples in registers
# or cut planes into column tiles, which a uniformly drawn P seldom reaches
for i in range(12 * SCALE):
    _g = np.random.default_rng(550000 + i)
    C = log_uniform(_g, 33, 700)
    ND_CASES.append((min(4 * log_uniform(_g, 2, 255), max(4, ((BUDGET >> 1) // C) & ~3)), C, log_uniform(_g, 1, 6),
                     int(_g.integers(0, 4))))


@pytest.mark.parametrize("P,C,N,offset", ND_CASES)
def test_nd_softmax_head_on_drawn_shapes(oracle, P, C, N, offset):
    print(f"case P={P} C={C} N={N} offset={offset}", flush=True)
    g = np.random.default_rng(P + 13 * C + N)
    n = P * C * N
    x = (1.5 * g.standard_normal(n)).astype(F32)
    lab = g.integers(0, C, P * N).astype(np.uint32)
    dy = g.standard_normal(P * N).astype(F32)
    old = g.standard_normal(n).astype(F32)
    xd, labd, dyd = dev(x, offset), dev(lab.view(np.int32), offset), dev(dy, offset)

    p_o = Guarded(n, offset)
    call("anode_gpu_softmax_nd_packed_f32", P, C, N, xd, p_o.view)
    p = p_o.get("softmax_nd")
    assert_close(p, oracle.softmax_nd(P, C, N, x, f64=True), "softmax_nd", abs_floor=1e-30)

    nll_o = Guarded(P * N, offset)
    call("anode_gpu_softmax_nd_cat_nll_packed_f32", P, C, N, p_o.view, labd, nll_o.view)
    nll = nll_o.get("nd nll")
    assert_close(nll, oracle.softmax_nd_cat_nll(P, C, N, p, lab, f64=True), "nd nll", abs_floor=1e-6)

    dx_o = Guarded(n, offset, init=old)
    call("anode_gpu_softmax_nd_cat_nll_bwd_packed_accumulate_f32", P, C, N, dyd, p_o.view, labd, dx_o.view)
    assert_bit_exact(dx_o.get("nd bwd"), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, p, lab, dx_in=old), "nd bwd acc")

    p2, n2 = Guarded(n, offset), Guarded(P * N, offset)
    call("anode_gpu_softmax_nd_cat_nll_fused_packed_f32", P, C, N, xd, labd, p2.view, n2.view)
    assert_bit_exact(p2.get("fused nd softmax"), p, "fused nd softmax")
    assert_bit_exact(n2.get("fused nd nll"), nll, "fused nd nll")
