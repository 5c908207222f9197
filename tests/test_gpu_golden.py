"""The GPU library against the committed fixtures of tests/golden/ (no oracle at run time): every reference entry
point at small ragged shapes, and the reference's own known answers (tests/test_gpu.rs:561-758).

Bit-exact where the arithmetic is fully specified; |err| <= 1e-5 |ref| (+ the floors written below) against the fp64
columns for reductions, softmax, NLL and the transcendental maps.
"""
import json
import os

import numpy as np
import pytest

from gpu_util import F32, assert_bit_exact, assert_close, call, dev, empty, host, rms

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
EPS = 1e-5


@pytest.fixture(scope="module")
def G():
    with np.load(os.path.join(GOLDEN, "small_cases.npz")) as z:
        return {k: z[k] for k in z.files}


@pytest.fixture(scope="module")
def known():
    with open(os.path.join(GOLDEN, "reference_known_answers.json")) as f:
        return json.load(f)


def _shapes(G, prefix):
    return sorted({k.split("/")[0] for k in G if k.startswith(prefix)})


def test_batch_norm_fixtures(G):
    for k in _shapes(G, "bn_"):
        S, C, N = (int(v) for v in k[3:].split("x"))
        d = (S, C, N)
        g = lambda name: G[f"{k}/{name}"]
        x, dy = dev(g("x")), dev(g("dy"))
        mean, var = empty(C), empty(C)
        call("anode_gpu_batch_mean_3d1_packed_f32", *d, x, mean)
        assert_close(host(mean), g("mean64"), f"{k} mean")
        # downstream pieces take the fixture's fp32 statistics, so that each launch is compared on identical inputs
        mean_d, var_d = dev(g("mean")), dev(g("var"))
        call("anode_gpu_batch_var_3d1_packed_f32", *d, EPS, x, mean_d, var)
        assert_close(host(var), g("var64"), f"{k} var")
        y = empty(S * C * N)
        call("anode_gpu_batch_norm_3d1_packed_f32", *d, x, mean_d, var_d, y)
        assert_bit_exact(host(y), g("y"), f"{k} y")
        dx = empty(S * C * N)
        call("anode_gpu_batch_norm_bwd_3d1_packed_f32", *d, dy, var_d, dx)
        assert_bit_exact(host(dx), g("dx1"), f"{k} dx1")
        dmean, dvar = empty(C), empty(C)
        call("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", *d, dy, var_d, dmean)
        assert_close(host(dmean), g("dmean1_64"), f"{k} dmean1", abs_floor=1e-6 * rms(g("dmean1_64")))
        call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", *d, dy, x, mean_d, var_d, dvar)
        assert_close(host(dvar), g("dvar64"), f"{k} dvar", abs_floor=1e-6 * rms(g("dvar64")))
        dvar_d = dev(g("dvar"))
        dx = dev(g("dx1"))
        call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *d, dvar_d, x, mean_d, dx)
        assert_bit_exact(host(dx), g("dx2"), f"{k} dx2")
        dmean2 = dev(g("dmean2"))
        call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", *d, dmean2, dx)
        assert_bit_exact(host(dx), g("dx3"), f"{k} dx3")


def test_row_softmax_fixtures(G):
    for k in _shapes(G, "row_"):
        K, R = (int(v) for v in k[4:].split("x"))
        g = lambda name: G[f"{k}/{name}"]
        for sym in ("anode_gpu_softmax_packed_block_f32", "anode_gpu_softmax_packed_deterministic_f32"):
            p = empty(K * R)
            call(sym, K, R, dev(g("x")), p)
            assert_close(host(p), g("p64"), f"{k} p ({sym})")
        p_d, cat = dev(g("p")), dev(g("cat"))
        nll = empty(R)
        call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p_d, cat, nll)
        assert_close(host(nll), g("nll64"), f"{k} nll", abs_floor=1e-6)
        dx = empty(K * R)
        call("anode_gpu_softmax_cat_nll_bwd_packed_f32", K, R, dev(g("dy")), p_d, cat, dx)
        assert_bit_exact(host(dx), g("dx"), f"{k} dx")


def test_nd_softmax_fixtures(G):
    for k in _shapes(G, "nd_"):
        P, C, N = (int(v) for v in k[3:].split("x"))
        g = lambda name: G[f"{k}/{name}"]
        p = empty(P * C * N)
        call("anode_gpu_softmax_nd_packed_f32", P, C, N, dev(g("x")), p)
        assert_close(host(p), g("p64"), f"{k} p")
        p_d, cat = dev(g("p")), dev(g("cat"))
        nll = empty(P * N)
        call("anode_gpu_softmax_nd_cat_nll_packed_f32", P, C, N, p_d, cat, nll)
        assert_close(host(nll), g("nll64"), f"{k} nll", abs_floor=1e-6)
        dx = empty(P * C * N)
        call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dev(g("dy")), p_d, cat, dx)
        assert_bit_exact(host(dx), g("dx"), f"{k} dx")


def test_cast_and_one_hot_fixtures(G):
    import torch
    q = G["cast/q"]
    n = q.size
    u = empty(n, dtype=torch.int32)
    call("anode_gpu_upcast_u8_packed_u32", n, dev(q), u)
    assert np.array_equal(host(u).view(np.uint32), G["cast/upcast"])
    for lo, hi, key in ((0.0, 1.0, "cast/dequantize_0_1"), (-1.5, 2.25, "cast/dequantize_m1p5_2p25")):
        y = empty(n)
        call("anode_gpu_dequantize_u8_packed_f32", n, lo, hi, dev(q), y)
        assert_bit_exact(host(y), G[key], key)
    y = empty(5 * 7 * 3)
    call("anode_gpu_discrete_one_hot_3d1_packed_f32", 5, 7, 3, dev(G["one_hot/cat_5x7x3"]), y)
    assert_bit_exact(host(y), G["one_hot/y_5x7x3"], "one_hot")


EXACT_MAPS = ("copy", "modulus", "square", "sqrt", "positive_clip", "unit_step", "leaky_relu")
LIBM_MAPS = ("logistic", "normal_cdf", "tanh", "rcosh2")


def test_flat_map_fixtures(G):
    x, b = G["flat/x"], G["flat/b"]
    n = x.size
    for op in EXACT_MAPS + LIBM_MAPS:
        y = empty(n)
        if op == "leaky_relu":
            call("anode_gpu_leaky_relu_flat_map_f32", n, 0.125, dev(x), y)
        else:
            call(f"anode_gpu_{op}_flat_map_f32", n, dev(x), y)
        if op in EXACT_MAPS:
            assert_bit_exact(host(y), G[f"flat/{op}"], op)
        else:
            assert_close(host(y), G[f"flat/{op}64"], op, abs_floor=2e-7)
    for op in ("positive_clip_bwd", "logistic_bwd", "leaky_relu_bwd"):
        y = empty(n)
        if op == "leaky_relu_bwd":
            call("anode_gpu_leaky_relu_flat_map_bwd_f32", n, 0.125, dev(b), dev(x), y)
        else:
            call(f"anode_gpu_{op[:-4]}_flat_map_bwd_f32", n, dev(b), dev(x), y)
        assert_bit_exact(host(y), G[f"flat2/{op}"], op)
    y = empty(n)
    call("anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32", n, dev(b), dev(x), y)
    assert_bit_exact(host(y), G["flat2/copy_unit_step_join"], "flat_join")


def test_f1_fixtures(G):
    S, K, N = 23, 4, 3
    x, t = dev(G["f1/x"]), dev(G["f1/target"])
    y = empty(K * N)
    call("anode_gpu_smooth_negative_f1_loss_3d1_packed_f32", S, K, N, 1e-3, x, t, y)
    assert_close(host(y), G["f1/loss64"], "f1 loss")
    dx = empty(S * K * N)
    call("anode_gpu_smooth_negative_f1_loss_3d1_bwd_packed_f32", S, K, N, 1e-3, dev(G["f1/dy"]), x, t, dx)
    assert_bit_exact(host(dx), G["f1/dx"], "f1 bwd")


def test_reference_known_answers(known):
    k = known["softmax_cat_nll_adjoint"]
    K, R = k["K"], k["rows"]
    labels = np.array(k["labels"], np.uint32)
    for sym in ("anode_gpu_softmax_packed_block_f32", "anode_gpu_softmax_packed_deterministic_f32"):
        p = empty(K * R)
        call(sym, K, R, dev(np.zeros(K * R, F32)), p)
        assert np.all(host(p) == F32(known["softmax_zeros"]["p_expected_each"])), sym
    nll = empty(R)
    call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p, dev(labels), nll)
    ka = known["softmax_cat_nll"]
    assert np.allclose(host(nll), ka["nll_expected_each_f64"], rtol=ka["nll_rel_tol"], atol=0)
    dx = empty(K * R)
    call("anode_gpu_softmax_cat_nll_bwd_packed_f32", K, R, dev(np.full(R, k["dy_fill"], F32)), p, dev(labels), dx)
    want = np.full((R, K), k["dx_expected_off_label"], F32)
    want[np.arange(R), labels] = k["dx_expected_on_label"]
    assert np.array_equal(host(dx).reshape(R, K), want)

    ko = known["softmax_cat_nll_out_of_range"]
    call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p, dev(np.array(ko["labels"], np.uint32)), nll)
    assert list(np.isnan(host(nll))) == ko["nll_is_nan"]

    kd = known["dequantize_one"]
    y = empty(kd["count"])
    call("anode_gpu_dequantize_u8_packed_f32", kd["count"], kd["lo"], kd["hi"],
         dev(np.full(kd["count"], kd["code"], np.uint8)), y)
    assert np.all(host(y) == F32(1.0) / F32(255.0))

    kv = known["online_average"]
    xs, ys = dev(np.full(kv["count"], kv["x_fill"], F32)), dev(np.full(kv["count"], kv["y_fill"], F32))
    call("anode_gpu_online_average_packed_f32", kv["count"], kv["rate"], xs, ys)
    assert np.all(host(ys) == F32(kv["after_first"]))
    call("anode_gpu_online_average_packed_f32", kv["count"], kv["rate"], xs, ys)
    assert np.all(host(ys) == F32(kv["after_second"]))
