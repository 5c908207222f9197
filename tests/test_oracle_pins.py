"""Pins for the CPU oracle: before it is trusted as the checker of the HIP
kernels, every function is held against something it did not compute itself.

  * the reference's own known-answer tests (tests/test_gpu.rs:561-758);
  * what the mathematics fixes: closed forms, invariants, brute force over the
    reference's index order on tiny inputs, exact rational arithmetic;
  * float64 torch as an independent library (torch is this build's dependency,
    not the reference's).

Each check is chosen so that a plausible slip (a transposed dimension, a
dropped epsilon, a wrong sign, a biased/unbiased mix-up, a missing fused
multiply-add) fails it.
"""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

F32 = np.float32


def rng(seed=0):
    return np.random.default_rng(seed)


def nchw_to_flat(t):
    """A contiguous [N,C,*spatial] tensor is exactly the ABI's packed [S,C,N] array."""
    return np.ascontiguousarray(t).ravel()


# --------------------------------------------------------------------------
# reference known-answer tests
# --------------------------------------------------------------------------

def test_ref_softmax_zeros_is_exactly_one_over_32(oracle):
    # tests/test_gpu.rs:595-613: x = zeros[32 classes, 1 row] -> every p == 1.0/32.0 (assert_eq!)
    for bs in (32, 64, 1024):
        p = oracle.softmax(32, 1, np.zeros(32, F32), bs=bs)
        assert np.all(p == F32(1.0) / F32(32.0))
    p = oracle.softmax_nd(1, 32, 1, np.zeros(32, F32))
    assert np.all(p == F32(1.0) / F32(32.0))


def test_ref_softmax_cat_nll_labels_12_17(oracle):
    # tests/test_gpu.rs:615-649: zeros[32,2], labels [12,17] -> p == 1/32; nll = -logf(1/32)
    p = oracle.softmax(32, 2, np.zeros(64, F32))
    assert np.all(p == F32(1.0) / F32(32.0))
    nll = oracle.softmax_cat_nll(32, 2, p, np.array([12, 17], np.uint32))
    assert nll.dtype == F32
    np.testing.assert_allclose(nll, [math.log(32.0)] * 2, rtol=1e-7)
    assert np.all(nll == F32(3.4657359))


def test_ref_softmax_cat_nll_out_of_bounds_is_nan(oracle):
    # tests/test_gpu.rs:651-690: labels [12, 42] with 32 classes -> nll[1] NaN, the batch sum NaN
    p = oracle.softmax(32, 2, np.zeros(64, F32))
    nll = oracle.softmax_cat_nll(32, 2, p, np.array([12, 42], np.uint32))
    assert np.isfinite(nll[0]) and np.isnan(nll[1])
    assert np.isnan(nll.sum())
    nll64 = oracle.softmax_cat_nll(32, 2, p, np.array([12, 42], np.uint32), f64=True)
    assert np.isfinite(nll64[0]) and np.isnan(nll64[1])
    nd = oracle.softmax_nd_cat_nll(1, 32, 2, p, np.array([12, 42], np.uint32))
    assert np.isfinite(nd[0]) and np.isnan(nd[1])


def test_ref_softmax_cat_nll_sum_adjoint_closed_form(oracle):
    # tests/test_gpu.rs:692-736 builds d(sum nll)/dx: dy = 1, dx = 1/32 - [k == label]
    p = oracle.softmax(32, 2, np.zeros(64, F32))
    labels = np.array([12, 17], np.uint32)
    dx = oracle.softmax_cat_nll_bwd(32, 2, np.ones(2, F32), p, labels).reshape(2, 32)
    want = np.full((2, 32), F32(1.0) / F32(32.0), F32)
    want[0, 12] -= 1
    want[1, 17] -= 1
    assert np.array_equal(dx, want)


def test_ref_dequantize_ones_is_exactly_one_over_255(oracle):
    # tests/test_gpu.rs:738-758: u8 ones [32,32,3,1], lo 0, hi 1 -> y == 1.0/255.0 (assert_eq!)
    y = oracle.dequantize_u8(0.0, 1.0, np.ones(32 * 32 * 3, np.uint8))
    assert np.all(y == F32(1.0) / F32(255.0))


def test_ref_online_average_quarter_steps(oracle):
    # tests/test_gpu.rs:561-593: y0 = 0, x = 1, rate .25 -> 0.25 then 0.4375
    y = oracle.online_average(0.25, np.ones(1024, F32), np.zeros(1024, F32))
    assert np.all(y == F32(0.25))
    y = oracle.online_average(0.25, np.ones(1024, F32), y)
    assert np.all(y == F32(0.4375))


def test_online_discount_is_the_geometric_momentum_sum(oracle):
    # src/ops.rs:1425-1430: the momentum buffer starts at zero and takes y <- rate * y + grad each step.  With a
    # constant gradient of 1 and rate 1/2 the buffer is 2 - 2^(1-k): exactly representable, so a swapped operand
    # (rate * x + y gives k/2) or the running-average form (y + rate * (x - y) gives 1 - 2^-k) fails.
    y = np.zeros(257, F32)
    for k in range(1, 6):
        y = oracle.online_discount(0.5, np.ones(257, F32), y)
        assert np.all(y == F32(2.0 - 2.0 ** (1 - k)))
    # rate 0 forgets everything, rate 1 is a plain sum
    x = np.random.default_rng(3).standard_normal(257).astype(F32)
    assert np.array_equal(oracle.online_discount(0.0, x, y), x)
    assert np.array_equal(oracle.online_discount(1.0, x, y), (y + x).astype(F32))


# --------------------------------------------------------------------------
# bit-exact class: exact arithmetic and brute force
# --------------------------------------------------------------------------

def _round_fraction_to_f32(fr: Fraction) -> np.float32:
    """Correct round-to-nearest-even of an exact rational to binary32."""
    c = F32(float(fr))
    best = c
    for cand in (np.nextafter(c, F32(-np.inf)), np.nextafter(c, F32(np.inf))):
        d_c, d_b = abs(Fraction(float(cand)) - fr), abs(Fraction(float(best)) - fr)
        if d_c < d_b or (d_c == d_b and (int(cand.view(np.uint32)) & 1) == 0 and (int(best.view(np.uint32)) & 1) == 1):
            best = cand
    return best


@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-1.0, 1.0), (-0.5, 2.25), (0.1, 0.7), (-123.456, 789.01)])
def test_dequantize_all_codes_equal_single_rounded_fma(oracle, lo, hi):
    # quantize.cu:30-32 with nvcc's default contraction: y = fma(float(q), scale, lo), one rounding
    codes = np.arange(256, dtype=np.uint8)
    y = oracle.dequantize_u8(lo, hi, codes)
    scale = (F32(hi) - F32(lo)) / F32(255.0)
    want = np.array([_round_fraction_to_f32(Fraction(int(q)) * Fraction(float(scale)) + Fraction(float(F32(lo))))
                     for q in codes], F32)
    assert np.array_equal(y.view(np.uint32), want.view(np.uint32))
    assert y[0] == F32(lo)  # fma(0, s, lo) == lo


def test_dequantize_fused_differs_from_unfused_somewhere(oracle):
    # shows that the contraction choice is observable, i.e. that the pin above can fail
    codes = np.arange(256, dtype=np.uint8)
    a = oracle.dequantize_u8(0.1, 0.7, codes)
    b = oracle.dequantize_u8(0.1, 0.7, codes, fused=False)
    assert np.max(np.abs(a.astype(np.float64) - b.astype(np.float64))) <= 6e-8
    assert np.any(a != b)


def test_upcast_is_zero_extension(oracle):
    codes = np.arange(256, dtype=np.uint8)
    assert np.array_equal(oracle.upcast_u8(codes), np.arange(256, dtype=np.uint32))
    x = rng(1).integers(0, 256, 100003, dtype=np.uint8)
    assert np.array_equal(oracle.upcast_u8(x), x.astype(np.uint32))


def test_one_hot_brute_force_index_order(oracle):
    d0, K, d2 = 5, 4, 3
    lab = rng(2).integers(0, K + 2, d0 * d2).astype(np.uint32)  # includes labels >= K: no hit
    y = oracle.one_hot(d0, K, d2, lab)
    for i2 in range(d2):
        for k in range(K):
            for i0 in range(d0):
                want = 1.0 if lab[i0 + d0 * i2] == k else 0.0
                assert y[i0 + d0 * (k + K * i2)] == want
    assert y.sum() == np.count_nonzero(lab < K)


def test_gather_index_brute_force(oracle):
    K, R = 7, 5
    lab = np.array([0, 6, 7, 3, 100], np.uint32)
    idx = oracle.softmax_cat_gather_index(K, R, lab)
    for i in range(R):
        assert idx[i] == (lab[i] + K * i if lab[i] < K else np.iinfo(np.uint64).max)
    P, C, N = 4, 3, 2
    lab = rng(3).integers(0, C + 1, P * N).astype(np.uint32)
    idx = oracle.softmax_nd_cat_gather_index(P, C, N, lab)
    for n in range(N):
        for p in range(P):
            i = p + P * n
            assert idx[i] == (p + P * (lab[i] + C * n) if lab[i] < C else np.iinfo(np.uint64).max)


def test_arg_max_rules(oracle):
    # src/utils/mod.rs:31-41: first strict maximum from (-inf, 0); NaN never wins
    assert oracle.arg_max([1, 3, 3, 2]) == 1
    assert oracle.arg_max([-np.inf, -np.inf]) == 0
    assert oracle.arg_max([np.nan, 1.0, np.nan, 1.0]) == 1
    assert oracle.arg_max([np.nan, np.nan]) == 0
    assert oracle.arg_max(np.zeros(0, F32)) == 0
    assert oracle.arg_max([-1, -0.0, 0.0]) == 1  # -0.0 > -1; 0.0 > -0.0 is false
    x = rng(4).standard_normal((6, 10)).astype(F32)
    assert np.array_equal(oracle.arg_max_rows(10, 6, x.ravel()), x.argmax(1).astype(np.uint32))


SPECIALS = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.5, -2.25, 1e38, -1e38], F32)


def _bits(a):
    return np.asarray(a, F32).view(np.uint32)


def test_compare_multiply_maps_on_special_values(oracle):
    x = SPECIALS
    with np.errstate(invalid="ignore"):
        step = (x > 0).astype(F32)
        # flat_map.cu:175-178: ReLU by multiplication: -2.25 -> -0.0, -inf -> NaN, NaN -> NaN
        relu = oracle.flat_map("positive_clip", x)
        want = x * step
    assert np.array_equal(np.isnan(relu), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.array_equal(_bits(relu)[ok], _bits(want)[ok])
    assert np.signbit(relu[list(x).index(F32(-2.25))])  # negative zero, not +0
    assert np.isnan(relu[list(x).index(F32(-np.inf))])
    assert np.array_equal(_bits(oracle.flat_map("unit_step", x)), _bits(step))
    assert np.array_equal(_bits(oracle.flat_map("modulus", x))[ok], _bits(np.abs(x))[ok])
    assert np.array_equal(_bits(oracle.flat_map("copy", x)), _bits(x))
    with np.errstate(over="ignore", invalid="ignore"):
        sq = oracle.flat_map("square", x)
        assert np.array_equal(_bits(sq)[ok], _bits(x * x)[ok])
        # join and ReLU backward: a * float(b > 0)
        a = SPECIALS[::-1].copy()
        want = a * step
        for op in ("positive_clip_bwd", "copy_unit_step_join"):
            got = oracle.flat_map2(op, a, x)
            assert np.array_equal(np.isnan(got), np.isnan(want))
            assert np.array_equal(_bits(got)[~np.isnan(want)], _bits(want)[~np.isnan(want)])


def test_leaky_relu_and_logistic_bwd_formulas(oracle):
    x = rng(5).standard_normal(1000).astype(F32)
    dy = rng(6).standard_normal(1000).astype(F32)
    c = F32(0.01)
    y = oracle.flat_map("leaky_relu", x, c=c)
    assert np.array_equal(y, np.where(x > 0, x, c * x).astype(F32))
    dx = oracle.flat_map2("leaky_relu_bwd", dy, y, c=c)
    assert np.array_equal(dx, np.where(y > 0, dy, c * dy).astype(F32))
    s = oracle.flat_map("logistic", x)
    got = oracle.flat_map2("logistic_bwd", dy, s)
    assert np.array_equal(got, (dy * s) * (F32(1) - s))  # left-to-right, fp32 at each step


def test_transcendental_maps_against_float64(oracle):
    x = (rng(7).standard_normal(4096) * 3).astype(F32)
    x64 = x.astype(np.float64)
    ref = {
        "logistic": 1 / (1 + np.exp(-x64)),
        "tanh": np.tanh(x64),
        "rcosh2": 1 / np.cosh(x64) ** 2,
        "normal_cdf": 0.5 * (1 + np.vectorize(math.erf)(x64 / math.sqrt(2))),
        "sqrt": np.sqrt(np.abs(x64)),
    }
    for op, want in ref.items():
        arg = np.abs(x) if op == "sqrt" else x
        np.testing.assert_allclose(oracle.flat_map(op, arg), want, rtol=2e-6, atol=1e-7)
        np.testing.assert_allclose(oracle.flat_map(op, arg, f64=True), want, rtol=1e-12, atol=0)
    assert np.array_equal(oracle.flat_map("sqrt", np.abs(x)), np.sqrt(np.abs(x)))  # correctly rounded


# --------------------------------------------------------------------------
# batch norm: torch float64 as the independent check, plus invariants
# --------------------------------------------------------------------------

BN_SHAPES = [(2, 3, 5, 7), (4, 2, 1, 1), (3, 5, 7, 7), (2, 4, 33, 40)]


def _bn_case(shape, seed):
    g = rng(seed)
    x = (2 + 3 * g.standard_normal(shape)).astype(F32)
    dy = g.standard_normal(shape).astype(F32)
    N, C = shape[:2]
    S = int(np.prod(shape[2:]))
    return x, dy, S, C, N


@pytest.mark.parametrize("shape", BN_SHAPES)
def test_bn_forward_pieces_against_torch_float64(oracle, shape):
    x, _, S, C, N = _bn_case(shape, 10)
    eps = 1e-5
    xt = torch.from_numpy(x).double()
    dims = [0] + list(range(2, xt.ndim))
    mean_t = xt.mean(dims).numpy()
    var_t = xt.var(dims, unbiased=False).numpy()

    mean64 = oracle.batch_mean(S, C, N, nchw_to_flat(x), f64=True)
    np.testing.assert_allclose(mean64, mean_t, rtol=1e-13, atol=1e-14)
    mean32 = oracle.batch_mean(S, C, N, nchw_to_flat(x))
    np.testing.assert_allclose(mean32, mean_t, rtol=1e-5)

    # the reference's var is the BIASED variance PLUS epsilon, taken about the given fp32 mean
    var64 = oracle.batch_var(S, C, N, eps, nchw_to_flat(x), mean32, f64=True)
    shift = (mean32.astype(np.float64) - mean_t) ** 2
    np.testing.assert_allclose(var64, var_t + shift + np.float64(F32(eps)), rtol=1e-12)
    var32 = oracle.batch_var(S, C, N, eps, nchw_to_flat(x), mean32)
    np.testing.assert_allclose(var32, var_t + eps, rtol=1e-5)
    if S * N > 1:
        assert not np.allclose(var64, xt.var(dims, unbiased=True).numpy() + eps, rtol=1e-9)  # not unbiased

    y64 = oracle.batch_norm(S, C, N, nchw_to_flat(x), mean32, var32, f64=True).reshape(shape)
    y_t = torch.nn.functional.batch_norm(xt, None, None, training=True, eps=eps).numpy()
    np.testing.assert_allclose(y64, y_t, rtol=0, atol=2e-5)
    y32 = oracle.batch_norm(S, C, N, nchw_to_flat(x), mean32, var32).reshape(shape)
    np.testing.assert_allclose(y32, y64, rtol=1e-5, atol=1e-6)
    # invariants: per-channel mean of y ~ 0, biased variance of y ~ 1 - eps/var
    ych = np.moveaxis(y64, 1, 0).reshape(C, -1)
    np.testing.assert_allclose(ych.mean(1), 0, atol=1e-6)
    if S * N > 1:
        np.testing.assert_allclose(ych.var(1), 1 - eps / var32.astype(np.float64), rtol=1e-5)


@pytest.mark.parametrize("shape", BN_SHAPES[:1] + BN_SHAPES[2:])
def test_bn_backward_composite_equals_autograd_float64(oracle, shape):
    x, dy, S, C, N = _bn_case(shape, 11)
    eps = 1e-5
    xf, dyf = nchw_to_flat(x), nchw_to_flat(dy)
    mean = oracle.batch_mean(S, C, N, xf)
    var = oracle.batch_var(S, C, N, eps, xf, mean)

    # the recipe of src/ops_gpu.rs:4344-4352, 3997-4004, 3787-3795 in fp64
    dx = oracle.batch_norm_bwd(S, C, N, dyf, var, f64=True)
    dmean = oracle.batch_norm_bwd_mean(S, C, N, dyf, var, f64=True)
    dvar = oracle.batch_norm_bwd_var(S, C, N, dyf, xf, mean, var, f64=True)
    dvar32 = dvar.astype(F32)
    dx = dx + oracle.batch_var_bwd(S, C, N, dvar32, xf, mean, f64=True)
    dmean = dmean + oracle.batch_var_bwd_mean(S, C, N, dvar32, xf, mean, f64=True)
    dx = dx + oracle.batch_mean_bwd(S, C, N, dmean.astype(F32), f64=True)

    xt = torch.from_numpy(x).double().requires_grad_(True)
    yt = torch.nn.functional.batch_norm(xt, None, None, training=True, eps=eps)
    (gx,) = torch.autograd.grad(yt, xt, torch.from_numpy(dy).double())
    scale = np.abs(gx.numpy()).max()
    np.testing.assert_allclose(dx.reshape(shape), gx.numpy(), rtol=0, atol=2e-6 * scale)

    # each piece against its closed form
    v64 = var.astype(np.float64)
    rs = 1 / np.sqrt(v64)
    dych = np.moveaxis(dy.astype(np.float64), 1, 0).reshape(C, -1)
    xch = np.moveaxis(x.astype(np.float64), 1, 0).reshape(C, -1)
    np.testing.assert_allclose(oracle.batch_norm_bwd_mean(S, C, N, dyf, var, f64=True), -rs * dych.sum(1), rtol=1e-12)
    xc = xch - mean.astype(np.float64)[:, None]
    np.testing.assert_allclose(dvar, (dych * xc).sum(1) * (-0.5 * rs / v64), rtol=1e-11, atol=1e-13)
    np.testing.assert_allclose(oracle.batch_var_bwd_mean(S, C, N, dvar32, xf, mean, f64=True),
                               -2 * dvar32.astype(np.float64) * xc.sum(1) / (S * N), rtol=1e-9, atol=1e-12)
    # v2 uses the normalised output instead of (x, mean): same number
    y32 = oracle.batch_norm(S, C, N, xf, mean, var)
    v2 = oracle.batch_norm_bwd_var_v2(S, C, N, dyf, y32, var, f64=True)
    np.testing.assert_allclose(v2, dvar, rtol=2e-5, atol=1e-7 * np.abs(dvar).max())


def test_bn_index_order_brute_force(oracle):
    # a transposed (dim0, dim2) or a channel stride slip changes these
    d0, d1, d2 = 3, 4, 5
    x = rng(12).standard_normal(d0 * d1 * d2).astype(F32)
    want = np.zeros(d1)
    for i2 in range(d2):
        for i1 in range(d1):
            for i0 in range(d0):
                want[i1] += float(x[i0 + d0 * (i1 + d1 * i2)])
    np.testing.assert_allclose(oracle.batch_mean(d0, d1, d2, x, f64=True), want / (d0 * d2), rtol=1e-13)
    dm = rng(13).standard_normal(d1).astype(F32)
    dx = oracle.batch_mean_bwd(d0, d1, d2, dm)
    for idx in range(d0 * d1 * d2):
        assert dx[idx] == dm[(idx // d0) % d1] / F32(d0 * d2)


def test_bn_accumulate_variants_add_into_the_output(oracle):
    x, dy, S, C, N = _bn_case((3, 4, 5, 6), 14)
    xf, dyf = nchw_to_flat(x), nchw_to_flat(dy)
    mean = oracle.batch_mean(S, C, N, xf)
    var = oracle.batch_var(S, C, N, 1e-5, xf, mean)
    old = rng(15).standard_normal(xf.size).astype(F32)
    oldc = rng(16).standard_normal(C).astype(F32)
    dv = rng(17).standard_normal(C).astype(F32)
    for f64 in (False, True):
        tol = dict(rtol=1e-12) if f64 else dict(rtol=1e-6, atol=1e-6)
        np.testing.assert_allclose(oracle.batch_norm_bwd(S, C, N, dyf, var, dx_in=old, f64=f64),
                                   old + oracle.batch_norm_bwd(S, C, N, dyf, var, f64=True), **tol)
        np.testing.assert_allclose(oracle.batch_var_bwd(S, C, N, dv, xf, mean, dx_in=old, f64=f64),
                                   old + oracle.batch_var_bwd(S, C, N, dv, xf, mean, f64=True), **tol)
        np.testing.assert_allclose(oracle.batch_mean_bwd(S, C, N, dv, dx_in=old, f64=f64),
                                   old + oracle.batch_mean_bwd(S, C, N, dv, f64=True), **tol)
        np.testing.assert_allclose(oracle.batch_norm_bwd_mean(S, C, N, dyf, var, dmean_in=oldc, f64=f64),
                                   oldc + oracle.batch_norm_bwd_mean(S, C, N, dyf, var, f64=True), **tol)
        np.testing.assert_allclose(oracle.batch_norm_bwd_var(S, C, N, dyf, xf, mean, var, dvar_in=oldc, f64=f64),
                                   oldc + oracle.batch_norm_bwd_var(S, C, N, dyf, xf, mean, var, f64=True), **tol)
        np.testing.assert_allclose(oracle.batch_var_bwd_mean(S, C, N, dv, xf, mean, dmean_in=oldc, f64=f64),
                                   oldc + oracle.batch_var_bwd_mean(S, C, N, dv, xf, mean, f64=True),
                                   rtol=tol["rtol"], atol=1e-6)


def _tile_tree_sum_threads(values, bs):
    """The reference's reduction as its threads execute it (common_reduce.cuh:22-31,
    batch_norm.cu:37-52), written out lane by lane in fp32."""
    acc = F32(0)
    n = len(values)
    for base in range(0, n, bs):
        cache = [F32(values[base + t]) if base + t < n else F32(0) for t in range(bs)]
        s = bs >> 1
        while s > 0:
            new = list(cache)
            for t in range(bs):  # every thread of the block, in lock step
                if s > t and s + t < bs:
                    new[t] = F32(cache[t] + cache[s + t])
            cache = new
            s >>= 1
        acc = F32(acc + cache[0])
    return acc


@pytest.mark.parametrize("bs", [4, 32, 128])
def test_f32ref_reduction_follows_the_reference_order(oracle, bs):
    d0, d1, d2 = 37, 2, 5
    x = (rng(18).standard_normal(d0 * d1 * d2) * 1000).astype(F32)
    got = oracle.batch_mean(d0, d1, d2, x, bs=bs)
    for c in range(d1):
        vals = [x[(i % d0) + d0 * (c + d1 * (i // d0))] for i in range(d0 * d2)]
        want = _tile_tree_sum_threads(vals, bs) / (F32(d0) * F32(d2))
        assert got[c] == want


def test_f32ref_reductions_agree_with_f64_within_tolerance(oracle):
    x, dy, S, C, N = _bn_case((8, 6, 14, 14), 19)
    xf, dyf = nchw_to_flat(x), nchw_to_flat(dy)
    mean = oracle.batch_mean(S, C, N, xf)
    var = oracle.batch_var(S, C, N, 1e-5, xf, mean)
    np.testing.assert_allclose(oracle.batch_norm_bwd_mean(S, C, N, dyf, var),
                               oracle.batch_norm_bwd_mean(S, C, N, dyf, var, f64=True), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(oracle.batch_norm_bwd_var(S, C, N, dyf, xf, mean, var),
                               oracle.batch_norm_bwd_var(S, C, N, dyf, xf, mean, var, f64=True), rtol=1e-4, atol=1e-5)


# --------------------------------------------------------------------------
# softmax / NLL
# --------------------------------------------------------------------------

@pytest.mark.parametrize("K,R", [(1, 3), (10, 32), (33, 7), (1000, 5), (2500, 2)])
def test_softmax_rows_against_torch_float64(oracle, K, R):
    x = (2 * rng(20).standard_normal((R, K))).astype(F32)
    want = torch.softmax(torch.from_numpy(x).double(), dim=1).numpy()
    p64 = oracle.softmax(K, R, x.ravel(), f64=True).reshape(R, K)
    np.testing.assert_allclose(p64, want, rtol=1e-13)
    for bs in (32, 1024):
        p32 = oracle.softmax(K, R, x.ravel(), bs=bs).reshape(R, K)
        np.testing.assert_allclose(p32, want, rtol=1e-5, atol=1e-30)
        np.testing.assert_allclose(p32.astype(np.float64).sum(1), 1, atol=1e-5)
    # shift invariance (exact for a power-of-two shift of these magnitudes would not hold; use tolerance)
    shifted = oracle.softmax(K, R, (x + F32(8)).ravel(), f64=True).reshape(R, K)
    np.testing.assert_allclose(shifted, want, rtol=1e-5)


def test_softmax_nll_and_bwd_against_torch(oracle):
    K, R = 10, 32
    x = rng(21).standard_normal((R, K)).astype(F32)
    lab = rng(22).integers(0, K, R).astype(np.uint32)
    p = oracle.softmax(K, R, x.ravel())
    nll64 = oracle.softmax_cat_nll(K, R, p, lab, f64=True)
    xt = torch.from_numpy(x).double().requires_grad_(True)
    ce = torch.nn.functional.cross_entropy(xt, torch.from_numpy(lab.astype(np.int64)), reduction="none")
    np.testing.assert_allclose(nll64, ce.detach().numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(oracle.softmax_cat_nll(K, R, p, lab), nll64, rtol=1e-6, atol=1e-7)
    dy = rng(23).standard_normal(R).astype(F32)
    (gx,) = torch.autograd.grad(ce, xt, torch.from_numpy(dy).double())
    dx64 = oracle.softmax_cat_nll_bwd(K, R, dy, p, lab, f64=True).reshape(R, K)
    np.testing.assert_allclose(dx64, gx.numpy(), rtol=0, atol=1e-6)
    dx32 = oracle.softmax_cat_nll_bwd(K, R, dy, p, lab).reshape(R, K)
    np.testing.assert_allclose(dx32, dx64, rtol=1e-6, atol=1e-7)
    # out-of-range label: no one-hot hit, gradient is dy * p, unmasked (softmax.cu:188-193)
    bad = lab.copy()
    bad[3] = 255
    dxb = oracle.softmax_cat_nll_bwd(K, R, dy, p, bad).reshape(R, K)
    assert np.array_equal(dxb[3], dy[3] * p.reshape(R, K)[3])
    # accumulate adds into dx
    old = rng(24).standard_normal(R * K).astype(F32)
    acc = oracle.softmax_cat_nll_bwd(K, R, dy, p, lab, dx_in=old, f64=True)
    np.testing.assert_allclose(acc, old + dx64.ravel(), rtol=1e-13)


def test_softmax_nd_against_torch_and_row_form(oracle):
    N, C, H, W = 2, 19, 6, 8
    P = H * W
    x = rng(25).standard_normal((N, C, H, W)).astype(F32)
    lab = rng(26).integers(0, C, (N, H, W)).astype(np.uint32)
    lab[0, 0, :3] = 255  # ignore-index style labels: NaN nll, unmasked gradient in the reference
    want = torch.softmax(torch.from_numpy(x).double(), dim=1).numpy()
    p64 = oracle.softmax_nd(P, C, N, x.ravel(), f64=True).reshape(x.shape)
    np.testing.assert_allclose(p64, want, rtol=1e-13)
    p32 = oracle.softmax_nd(P, C, N, x.ravel())
    np.testing.assert_allclose(p32.reshape(x.shape), want, rtol=1e-5)
    # with P == 1 the n-d form is the row form
    xr = rng(27).standard_normal((5, 7)).astype(F32)
    assert np.array_equal(oracle.softmax_nd(1, 7, 5, xr.ravel()), oracle.softmax(7, 5, xr.ravel(), bs=8)) or \
        np.allclose(oracle.softmax_nd(1, 7, 5, xr.ravel()), oracle.softmax(7, 5, xr.ravel()), rtol=1e-6)

    nll = oracle.softmax_nd_cat_nll(P, C, N, p32, lab.ravel(), f64=True).reshape(N, H, W)
    bad = lab == 255
    assert np.all(np.isnan(nll[bad])) and not np.any(np.isnan(nll[~bad]))
    ce = torch.nn.functional.cross_entropy(torch.from_numpy(x).double(),
                                           torch.from_numpy(np.where(bad, 0, lab).astype(np.int64)), reduction="none").numpy()
    np.testing.assert_allclose(nll[~bad], ce[~bad], rtol=1e-5, atol=1e-6)

    dy = rng(28).standard_normal((N, H, W)).astype(F32)
    dx = oracle.softmax_nd_cat_nll_bwd(P, C, N, dy.ravel(), p32, lab.ravel(), f64=True).reshape(x.shape)
    pr = p32.reshape(x.shape).astype(np.float64)
    onehot = (np.arange(C)[None, :, None, None] == lab[:, None]).astype(np.float64)
    np.testing.assert_allclose(dx, dy[:, None].astype(np.float64) * (pr - onehot), rtol=1e-13)
    assert np.allclose(dx[0, :, 0, 0], dy[0, 0, 0] * pr[0, :, 0, 0])  # bad label: unmasked dy * p


# --------------------------------------------------------------------------
# F1, additive symbols
# --------------------------------------------------------------------------

def test_f1_loss_brute_force(oracle):
    d0, K, N = 50, 3, 2
    g = rng(29)
    x = g.random(d0 * K * N).astype(F32)
    t = (g.random(d0 * K * N) > 0.5).astype(F32)
    eps = 1e-3
    want = np.zeros(K * N)
    for r in range(K * N):
        num = sum(float(x[r * d0 + i]) * float(t[r * d0 + i]) for i in range(d0))
        den = sum(float(x[r * d0 + i]) + float(t[r * d0 + i]) for i in range(d0))
        want[r] = -(2 * num + float(F32(eps))) / (den + float(F32(eps)))
    np.testing.assert_allclose(oracle.f1_loss(d0, K, N, eps, x, t, f64=True), want, rtol=1e-13)
    np.testing.assert_allclose(oracle.f1_loss(d0, K, N, eps, x, t, bs=64), want, rtol=1e-5)
    dy = g.standard_normal(K * N).astype(F32)
    e = float(F32(eps))
    x64, t64 = x.astype(np.float64), t.astype(np.float64)
    want_bwd = np.repeat(dy.astype(np.float64), d0) * -(2 * t64 * (t64 + e) - e) / (x64 + t64 + e) ** 2
    np.testing.assert_allclose(oracle.f1_loss_bwd(d0, K, N, eps, dy, x, t, f64=True), want_bwd, rtol=1e-13)
    np.testing.assert_allclose(oracle.f1_loss_bwd(d0, K, N, eps, dy, x, t), want_bwd, rtol=1e-5, atol=1e-6)


def test_quantize_is_the_inverse_of_dequantize(oracle):
    for lo, hi in [(0.0, 1.0), (-1.0, 1.0), (-3.5, 2.25)]:
        codes = np.arange(256, dtype=np.uint8)
        assert np.array_equal(oracle.quantize_u8(lo, hi, oracle.dequantize_u8(lo, hi, codes)), codes)
    # round-half-even at exact half-way points (lo 0, hi 255 -> scale exactly 1)
    x = np.array([0.5, 1.5, 2.5, 3.5, 254.5, 255.5, -0.5, -7, 300, np.nan, np.inf, -np.inf], F32)
    assert list(oracle.quantize_u8(0.0, 255.0, x)) == [0, 2, 2, 4, 254, 255, 0, 0, 255, 0, 255, 0]
    z = np.sort(rng(30).standard_normal(10000).astype(F32))
    q = oracle.quantize_u8(-4.0, 4.0, z)
    assert np.all(np.diff(q.astype(np.int32)) >= 0)  # monotone


def test_bcast_affine_and_mean_var(oracle):
    inner, bc, outer = 6, 3, 4
    g = rng(31)
    lx, sh = g.standard_normal(bc).astype(F32), g.standard_normal(bc).astype(F32)
    rx = g.standard_normal(inner * bc * outer).astype(F32)
    y = oracle.bcast_flat_mult_add(inner, bc, outer, lx, rx, sh).reshape(outer, bc, inner)
    want = lx.astype(np.float64)[None, :, None] * rx.reshape(outer, bc, inner) + sh.astype(np.float64)[None, :, None]
    np.testing.assert_allclose(y, want, rtol=1e-6, atol=1e-7)
    y2 = oracle.bcast_flat_mult_add(inner, bc, outer, lx, rx).reshape(outer, bc, inner)
    assert np.array_equal(y2, lx[None, :, None] * rx.reshape(outer, bc, inner))
    q = g.integers(0, 256, inner * bc * outer).astype(np.uint8)
    y3 = oracle.bcast_dequantize_u8(inner, bc, outer, lx, sh, q).reshape(outer, bc, inner)
    want3 = lx.astype(np.float64)[None, :, None] * q.reshape(outer, bc, inner) + sh.astype(np.float64)[None, :, None]
    np.testing.assert_allclose(y3, want3, rtol=1e-6, atol=1e-6)
    x = (2 + 3 * g.standard_normal((4, 3, 5, 5))).astype(F32)
    m, v = oracle.batch_mean_var(25, 3, 4, 1e-5, x.ravel())
    xt = torch.from_numpy(x).double()
    np.testing.assert_allclose(m, xt.mean((0, 2, 3)).numpy(), rtol=1e-13)
    np.testing.assert_allclose(v, xt.var((0, 2, 3), unbiased=False).numpy() + float(F32(1e-5)), rtol=1e-12)


# --------------------------------------------------------------------------
# the additive reductions / maps and the gpudevicemem neighbours
# --------------------------------------------------------------------------

def test_channel_sum_triple_loop_on_a_lopsided_array(oracle):
    # the commented-out declarations lib.h:408-430: y[b] = sum over a and c of x[a,b,c] (or of its square).
    # All three extents differ, so a transposed extent or a sum over the wrong axis lands on other numbers.
    d0, d1, d2 = 5, 3, 2
    x = (rng(41).standard_normal(d0 * d1 * d2) * 3 + 1).astype(F32)
    plain = [0.0] * d1
    squares = [0.0] * d1
    for c in range(d2):
        for b in range(d1):
            for a in range(d0):
                v = float(x[a + d0 * (b + d1 * c)])
                plain[b] += v
                squares[b] += v * v
    np.testing.assert_allclose(oracle.channel_sum(d0, d1, d2, x), plain, rtol=1e-14)
    np.testing.assert_allclose(oracle.channel_sum(d0, d1, d2, x, square=True), squares, rtol=1e-14)
    assert not np.allclose(plain, squares)
    # integers: the sums are exact, whatever the order
    xi = np.arange(d0 * d1 * d2, dtype=F32)
    t = xi.reshape(d2, d1, d0).astype(np.float64)
    assert np.array_equal(oracle.channel_sum(d0, d1, d2, xi), t.sum((0, 2)))
    assert np.array_equal(oracle.channel_sum(d0, d1, d2, xi, square=True), (t * t).sum((0, 2)))
    # against torch float64 on an NCHW view
    xt = torch.from_numpy(x.reshape(d2, d1, d0)).double()
    np.testing.assert_allclose(oracle.channel_sum(d0, d1, d2, x), xt.sum((0, 2)).numpy(), rtol=1e-14)


def test_batch_norm_affine_is_one_fma_over_the_pinned_batch_norm(oracle):
    # y = fma(batch_norm(x)[c], gamma[c], beta[c]): composed from batch_norm (pinned against torch float64 above)
    # with exact rational arithmetic for the one rounding, and against torch's own affine batch norm.
    N, C, H, W = 3, 4, 2, 5
    S = H * W
    g = rng(42)
    x = (2 + 3 * g.standard_normal((N, C, H, W))).astype(F32)
    gamma = g.uniform(0.5, 1.5, C).astype(F32)
    beta = (0.1 * g.standard_normal(C)).astype(F32)
    eps = F32(1e-5)
    xf = nchw_to_flat(x)
    mean = oracle.batch_mean(S, C, N, xf)
    var = oracle.batch_var(S, C, N, eps, xf, mean)
    yn = oracle.batch_norm(S, C, N, xf, mean, var)
    got = oracle.batch_norm_affine(S, C, N, xf, mean, var, gamma, beta)
    assert got.dtype == F32
    want = np.empty_like(got)
    for i in range(got.size):
        c = (i // S) % C
        want[i] = _round_fraction_to_f32(Fraction(float(yn[i])) * Fraction(float(gamma[c])) + Fraction(float(beta[c])))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # an unfused multiply-then-add differs somewhere, so the pin above can fail
    unfused = (yn * gamma[(np.arange(got.size) // S) % C] + beta[(np.arange(got.size) // S) % C]).astype(F32)
    assert np.any(unfused != got)
    # torch float64: the reference stores var = biased variance + eps, torch adds eps itself
    xt = torch.from_numpy(x).double()
    ref = torch.nn.functional.batch_norm(xt, None, None, torch.from_numpy(gamma).double(), torch.from_numpy(beta).double(),
                                         training=True, eps=float(eps)).numpy().ravel()
    m64, v64 = oracle.batch_mean_var(S, C, N, eps, xf)
    got64 = oracle.batch_norm_affine(S, C, N, xf, m64.astype(F32), v64.astype(F32), gamma, beta, f64=True)
    np.testing.assert_allclose(got64, ref, rtol=2e-6, atol=2e-6)   # mean / var were rounded to f32 on the way in
    np.testing.assert_allclose(got, ref, rtol=1e-5, atol=1e-5)
    # gamma 1, beta 0 is batch_norm itself, bit for bit (fma(y, 1, 0) == y)
    same = oracle.batch_norm_affine(S, C, N, xf, mean, var, np.ones(C, F32), np.zeros(C, F32))
    assert np.array_equal(same.view(np.uint32), (yn + F32(0)).view(np.uint32))
    # swapped gamma / beta would give this instead
    swapped = oracle.batch_norm_affine(S, C, N, xf, mean, var, beta, gamma)
    assert not np.allclose(swapped, got)


def test_sum_packed_ten_ones_and_float64_sum(oracle):
    # tests/test_gpu.rs:302-353: ten arrays of ones joined by a sum give 10.0 in every element; the packed sum of
    # ten ones is the same 10.0
    assert oracle.sum_packed(np.ones(10, F32)) == 10.0
    assert oracle.sum_packed(np.zeros(0, F32)) == 0.0
    x = (rng(43).standard_normal(100003) * 1e3).astype(F32)
    assert oracle.sum_packed(x) == pytest.approx(math.fsum(float(v) for v in x), rel=1e-15)
    # a sum carried in float32 is off by far more than that
    assert abs(float(np.cumsum(x, dtype=F32)[-1]) - math.fsum(float(v) for v in x)) > 1e-3
    # integers below 2^24: exact
    assert oracle.sum_packed(np.arange(5000, dtype=F32)) == 5000 * 4999 / 2


def test_online_add_is_a_single_rounded_fma(oracle):
    # src/ops_gpu.rs:5886: y <- y + rate * x.  Exact rationals: one rounding, operands in this order
    g = rng(44)
    x = g.standard_normal(300).astype(F32)
    y = g.standard_normal(300).astype(F32)
    for rate in (0.1, -0.75, 1e-3, 3.0):
        got = oracle.online_add(rate, x, y)
        r = Fraction(float(F32(rate)))
        want = np.array([_round_fraction_to_f32(r * Fraction(float(a)) + Fraction(float(b))) for a, b in zip(x, y)], F32)
        assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
        unfused = (F32(rate) * x + y).astype(F32)
        assert np.max(np.abs(unfused.astype(np.float64) - got)) <= 1e-6
    assert np.any((F32(0.1) * x + y).astype(F32) != oracle.online_add(0.1, x, y))   # the fusion is observable
    # it is not the running-average form (rate 1 would return x) nor the discount form (rate 0 would return x)
    assert np.array_equal(oracle.online_add(1.0, x, y), (x + y).astype(F32))
    assert np.array_equal(oracle.online_add(0.0, x, y), y)
    # three steps of +0.25 from zero: 0.25, 0.5, 0.75 exactly
    acc = np.zeros(17, F32)
    for k in range(1, 4):
        acc = oracle.online_add(0.25, np.ones(17, F32), acc)
        assert np.all(acc == F32(0.25 * k))


def test_flat_bcast_rdiv_brute_force_ieee_division(oracle):
    # src/ops_gpu.rs:9592 (I1ab, I2b -> Oab): y[a,b] = x[a,b] / r[b], a fastest
    inner, outer = 7, 5
    g = rng(45)
    x = g.standard_normal(inner * outer).astype(F32)
    r = g.uniform(0.5, 3.0, outer).astype(F32)
    got = oracle.flat_bcast_rdiv(inner, outer, x, r)
    want = np.empty(inner * outer, F32)
    for b in range(outer):
        for a in range(inner):
            want[a + inner * b] = _round_fraction_to_f32(Fraction(float(x[a + inner * b])) / Fraction(float(r[b])))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # multiplying by a rounded reciprocal is not the same thing
    recip = (x.reshape(outer, inner) * (F32(1) / r)[:, None]).astype(F32).ravel()
    xs = g.standard_normal(4096 * 3).astype(F32)
    rs = g.uniform(0.5, 3.0, 3).astype(F32)
    assert np.any(oracle.flat_bcast_rdiv(4096, 3, xs, rs) != (xs.reshape(3, 4096) * (F32(1) / rs)[:, None]).astype(F32).ravel())
    assert np.max(np.abs(recip.astype(np.float64) - got)) < 1e-6
    # a divisor indexed by the inner index would divide by the wrong element
    wrong = (x.reshape(outer, inner) / np.resize(r, inner)[None, :]).astype(F32).ravel()
    assert not np.array_equal(wrong, got)
    # special values: x/inf = 0, x/0 = inf with the sign of x, 0/0 = NaN
    sv = oracle.flat_bcast_rdiv(2, 3, np.array([1, -1, 2, -2, 0, 3], F32), np.array([np.inf, 0.0, 0.0], F32))
    assert sv[0] == 0 and sv[1] == 0 and np.signbit(sv[1]) and sv[2] == np.inf and sv[3] == -np.inf
    assert np.isnan(sv[4]) and sv[5] == np.inf
