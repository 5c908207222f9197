"""GPU parity for the additive entry points (no kernel in the reference: pinned
by closed form, by the oracle's restatement, and -- for the fused ones -- by
equality with the sequence of reference-ABI launches they replace)."""
import numpy as np
import pytest
import torch

from gpu_util import F32, assert_bit_exact, assert_close, call, dev, empty, host, rms

pytestmark = pytest.mark.gpu

LENGTHS = [1, 3, 4, 5, 15, 16, 17, 1023, 1024, 4095, 4096, 4099, 4111, 8191, (1 << 20) + 2]


@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-1.0, 1.0), (-3.5, 2.25), (0.0, 255.0)])
def test_quantize_u8(oracle, lo, hi):
    g = np.random.default_rng(0)
    codes = np.arange(256, dtype=np.uint8)
    deq = empty(256)
    call("anode_gpu_dequantize_u8_packed_f32", 256, lo, hi, dev(codes), deq)
    back = empty(256, dtype=torch.uint8)
    call("anode_gpu_quantize_u8_packed_f32", 256, lo, hi, deq, back)
    assert np.array_equal(host(back), codes)  # quantize(dequantize(q)) == q for every code
    for n in LENGTHS:
        x = (lo + (hi - lo) * (g.random(n) * 1.2 - 0.1)).astype(F32)
        k = min(n, 6)
        x[:k] = np.array([np.nan, np.inf, -np.inf, lo, hi, (lo + hi) / 2], F32)[:k]
        for off_in, off_out in [(0, 0), (1, 0), (0, 1), (0, 4)]:
            y = empty(n, dtype=torch.uint8, offset=off_out)
            call("anode_gpu_quantize_u8_packed_f32", n, lo, hi, dev(x, off_in), y)
            assert_bit_exact(host(y), oracle.quantize_u8(lo, hi, x), f"quantize n={n}")
    # half-way cases round to even (scale is exactly 1 here)
    x = np.array([0.5, 1.5, 2.5, 3.5, 254.5, 255.5, -0.5], F32)
    y = empty(7, dtype=torch.uint8)
    call("anode_gpu_quantize_u8_packed_f32", 7, 0.0, 255.0, dev(x), y)
    assert list(host(y)) == [0, 2, 2, 4, 254, 255, 0]


@pytest.mark.parametrize("inner,bc,outer", [(50176, 3, 4), (49, 20, 3), (1, 7, 5), (5, 3, 2), (4096, 2, 3)])
def test_bcast_affine_family(oracle, inner, bc, outer):
    g = np.random.default_rng(inner)
    n = inner * bc * outer
    lx, sh = g.standard_normal(bc).astype(F32), g.standard_normal(bc).astype(F32)
    rx = g.standard_normal(n).astype(F32)
    for offset in (0, 1):
        y = empty(n, offset=offset)
        call("anode_gpu_bcast_flat_mult_add_I1b_I2abc_Oabc_packed_f32", inner, bc, outer, dev(lx), dev(rx, offset), dev(sh), y)
        assert_bit_exact(host(y), oracle.bcast_flat_mult_add(inner, bc, outer, lx, rx, sh), "mult_add abc")
        call("anode_gpu_bcast_flat_mult_I1b_I2abc_Oabc_packed_f32", inner, bc, outer, dev(lx), dev(rx, offset), y)
        assert_bit_exact(host(y), oracle.bcast_flat_mult_add(inner, bc, outer, lx, rx), "mult abc")
        q = g.integers(0, 256, n, dtype=np.uint8)
        call("anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32", inner, bc, outer, dev(lx), dev(sh), dev(q, offset), y)
        assert_bit_exact(host(y), oracle.bcast_dequantize_u8(inner, bc, outer, lx, sh, q), "bcast dequantize")
    # two-index forms are the outer_dim == 1 case
    m = inner * bc
    y = empty(m)
    call("anode_gpu_bcast_flat_mult_add_I1b_I2ab_Oab_packed_f32", inner, bc, dev(lx), dev(rx[:m]), dev(sh), y)
    assert_bit_exact(host(y), oracle.bcast_flat_mult_add(inner, bc, 1, lx, rx[:m], sh), "mult_add ab")
    call("anode_gpu_bcast_flat_mult_I1b_I2ab_Oab_packed_f32", inner, bc, dev(lx), dev(rx[:m]), y)
    assert_bit_exact(host(y), oracle.bcast_flat_mult_add(inner, bc, 1, lx, rx[:m]), "mult ab")
    # flat forms
    a, b, c = rx[:m], rx[::-1][:m].copy(), g.standard_normal(m).astype(F32)
    call("anode_gpu_flat_mult_f32", m, dev(a), dev(b), y)
    assert_bit_exact(host(y), a * b, "flat_mult")
    call("anode_gpu_flat_mult_add_f32", m, dev(a), dev(b), dev(c), y)
    want = (a.astype(np.float64) * b.astype(np.float64) + c.astype(np.float64))
    assert_close(host(y), want, "flat_mult_add", rel=1e-6, abs_floor=1e-7)


def test_imagenet_normalisation_is_dequantize_then_affine(oracle):
    # config 1: u8 image batch -> float, normalised per channel with ImageNet statistics
    n_img, C, S = 8, 3, 224 * 224
    q = np.random.default_rng(1).integers(0, 256, n_img * C * S, dtype=np.uint8)
    mean = np.array([0.485, 0.456, 0.406], F32)
    std = np.array([0.229, 0.224, 0.225], F32)
    a = (F32(1.0) / (F32(255.0) * std)).astype(F32)
    b = (-mean / std).astype(F32)
    y = empty(q.size)
    call("anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32", S, C, n_img, dev(a), dev(b), dev(q), y)
    want = (q.reshape(n_img, C, S).astype(np.float64) / 255 - mean[None, :, None]) / std[None, :, None]
    assert_close(host(y).reshape(n_img, C, S), want, "imagenet normalisation", rel=1e-5, abs_floor=1e-6)


@pytest.mark.parametrize("S,C,N", [(784, 16, 32), (49, 300, 4), (1, 37, 11), (5000, 3, 4), (40000, 2, 1), (7, 513, 2)])
def test_channel_sums_and_mean_var(oracle, S, C, N):
    g = np.random.default_rng(S + C)
    x = (1000 + 3 * g.standard_normal(S * C * N)).astype(F32)  # a large offset: the single pass must stay accurate
    for offset in (0, 1):
        xd = dev(x, offset)
        y = empty(C, offset=offset)
        call("anode_gpu_sum_Iabc_Ob_packed_deterministic_f32", S, C, N, xd, y)
        assert_close(host(y), oracle.channel_sum(S, C, N, x), "sum_Iabc_Ob")
        call("anode_gpu_square_sum_Iabc_Ob_packed_deterministic_f32", S, C, N, xd, y)
        assert_close(host(y), oracle.channel_sum(S, C, N, x, square=True), "square_sum_Iabc_Ob")
        mean, var = empty(C, offset=offset), empty(C, offset=offset)
        call("anode_gpu_batch_mean_var_3d1_packed_f32", S, C, N, 1e-5, xd, mean, var)
        m64, v64 = oracle.batch_mean_var(S, C, N, 1e-5, x)
        assert_close(host(mean), m64, "mean of mean_var")
        assert_close(host(var), v64, "var of mean_var")
        # agrees with the two-launch reference path within the tolerance class
        m2, v2 = empty(C), empty(C)
        call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, xd, m2)
        call("anode_gpu_batch_var_3d1_packed_f32", S, C, N, 1e-5, xd, m2, v2)
        assert_bit_exact(host(mean), host(m2), "mean: one pass vs two")
        assert_close(host(var), host(v2), "var: one pass vs two")
        # with the running statistics moved in the same launch: the bits of mean_var followed by two online_average
        g2 = np.random.default_rng(C)
        rm0, rv0 = g2.standard_normal(C).astype(F32), g2.uniform(0.5, 2.0, C).astype(F32)
        rm1, rv1 = dev(rm0, offset), dev(rv0, offset)
        call("anode_gpu_online_average_packed_f32", C, 0.1, mean, rm1)
        call("anode_gpu_online_average_packed_f32", C, 0.1, var, rv1)
        m3, v3, rm2, rv2 = empty(C, offset=offset), empty(C, offset=offset), dev(rm0, offset), dev(rv0, offset)
        call("anode_gpu_batch_mean_var_online_3d1_packed_f32", S, C, N, 1e-5, 0.1, xd, m3, v3, rm2, rv2)
        assert_bit_exact(host(m3), host(mean), "mean_var_online mean")
        assert_bit_exact(host(v3), host(var), "mean_var_online var")
        assert_bit_exact(host(rm2), host(rm1), "running mean")
        assert_bit_exact(host(rv2), host(rv1), "running var")
        assert_bit_exact(host(rm2), oracle.online_average(0.1, host(mean), rm0), "running mean vs oracle")
    xs = x[:S * C]
    y = empty(C)
    call("anode_gpu_sum_Iab_Ob_packed_deterministic_f32", S, C, dev(xs), y)
    assert_close(host(y), oracle.channel_sum(S, C, 1, xs), "sum_Iab_Ob")


@pytest.mark.parametrize("S,C,N", [(784, 16, 8), (49, 20, 6), (5000, 3, 4), (1, 37, 11), (12544, 4, 4)])
@pytest.mark.parametrize("masked", [False, True])
def test_fused_batch_norm_equals_the_launch_sequence(oracle, S, C, N, masked):
    g = np.random.default_rng(S * 3 + C)
    n = S * C * N
    x = (2 + 3 * g.standard_normal(n)).astype(F32)
    dy = g.standard_normal(n).astype(F32)
    gamma = (0.5 + g.random(C)).astype(F32)
    beta = (0.1 * g.standard_normal(C)).astype(F32)
    old = g.standard_normal(n).astype(F32)
    d = (S, C, N)
    for offset in (0, 1):
        xd, dyd = dev(x, offset), dev(dy, offset)
        mean, var = empty(C), empty(C)
        call("anode_gpu_batch_mean_var_3d1_packed_f32", *d, 1e-5, xd, mean, var)
        mh, vh = host(mean), host(var)
        # forward: normalize + ReLU in one pass == batch_norm then positive_clip
        y_seq = empty(n, offset=offset)
        call("anode_gpu_batch_norm_3d1_packed_f32", *d, xd, mean, var, y_seq)
        call("anode_gpu_positive_clip_flat_map_f32", n, y_seq, y_seq)
        y_fused = empty(n, offset=offset)
        call("anode_gpu_batch_norm_positive_clip_3d1_packed_f32", *d, xd, mean, var, y_fused)
        assert_bit_exact(host(y_fused), host(y_seq), "norm+relu fused vs sequence")
        # forward: normalize + affine
        ya = empty(n, offset=offset)
        call("anode_gpu_batch_norm_affine_3d1_packed_f32", *d, xd, mean, var, dev(gamma), dev(beta), ya)
        assert_bit_exact(host(ya), oracle.batch_norm_affine(*d, x, mh, vh, gamma, beta), "norm+affine vs fp32")
        ref = oracle.batch_norm_affine(*d, x, mh, vh, gamma, beta, f64=True)
        assert_close(host(ya), ref, "norm+affine", abs_floor=1e-6 * rms(ref))

        # backward through (optional ReLU mask) + batch norm
        mask = y_fused if masked else None
        dy_eff = dyd
        if masked:
            dy_eff = empty(n, offset=offset)
            call("anode_gpu_positive_clip_flat_map_bwd_f32", n, dyd, y_fused, dy_eff)
        dmean_s, dvar_s, dx_s = empty(C), empty(C), empty(n, offset=offset)
        call("anode_gpu_batch_norm_bwd_3d1_packed_f32", *d, dy_eff, var, dx_s)
        call("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", *d, dy_eff, var, dmean_s)
        call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", *d, dy_eff, xd, mean, var, dvar_s)
        call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *d, dvar_s, xd, mean, dx_s)
        call("anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", *d, dvar_s, xd, mean, dmean_s)
        call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", *d, dmean_s, dx_s)

        dmean_f, dvar_f = empty(C), empty(C)
        call("anode_gpu_batch_norm_bwd_reduce_3d1_packed_f32", *d, dyd, xd, mean, var, mask, dmean_f, dvar_f)
        assert_close(host(dvar_f), host(dvar_s), "fused dvar vs sequence", abs_floor=1e-6 * rms(host(dvar_s)))
        assert_close(host(dmean_f), host(dmean_s), "fused dmean vs sequence", abs_floor=1e-6 * rms(host(dmean_s)))
        # given the same per-channel inputs, the fused map is the three launches bit for bit
        dx_f = empty(n, offset=offset)
        call("anode_gpu_batch_norm_bwd_apply_3d1_packed_f32", *d, dyd, xd, mean, var, dmean_s, dvar_s, mask, dx_f)
        assert_bit_exact(host(dx_f), host(dx_s), "fused dx vs sequence")
        # accumulate form: the sequence with an accumulating first writer
        dx_sa = dev(old, offset)
        call("anode_gpu_batch_norm_bwd_3d1_packed_accumulate_f32", *d, dy_eff, var, dx_sa)
        call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *d, dvar_s, xd, mean, dx_sa)
        call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", *d, dmean_s, dx_sa)
        dx_fa = dev(old, offset)
        call("anode_gpu_batch_norm_bwd_apply_3d1_packed_accumulate_f32", *d, dyd, xd, mean, var, dmean_s, dvar_s, mask, dx_fa)
        assert_bit_exact(host(dx_fa), host(dx_sa), "fused accumulate dx vs sequence")


@pytest.mark.parametrize("P,C,N", [(64, 19, 2), (2048, 19, 2), (5, 3, 4), (1, 10, 6), (16, 32, 2), (8, 40, 3), (100, 1, 3),
                                   (1300, 19, 3), (516, 24, 2), (1028, 2, 3), (12, 7, 5),
                                   (20, 48, 3), (24, 129, 2), (16, 200, 2), (8, 256, 3), (8, 300, 2), (520, 40, 2),
                                   # planes of 1024 pixels and more: the register and streaming kernels
                                   (1028, 8, 2), (1024, 32, 2), (1028, 48, 2), (1032, 65, 2), (1028, 129, 1),
                                   (1024, 192, 1), (1024, 256, 2), (1028, 300, 1), (1025, 19, 2), (1025, 40, 2),
                                   (1025, 130, 1),
                                   # short planes through the LDS tile, and its neighbours
                                   (196, 32, 9), (196, 41, 5), (196, 42, 3), (1023, 8, 3), (127, 64, 3), (127, 65, 3),
                                   (49, 20, 70), (7, 9, 1000), (4, 8, 4100), (2, 2, 9000), (512, 32, 3), (196, 64, 9),
                                   (9, 455, 6),
                                   # tiles of all classes of a run of pixels in LDS
                                   (64, 300, 3), (196, 150, 2), (1028, 200, 1), (20, 70, 5), (16, 944, 1), (1056, 256, 2),
                                   # samples of up to 63 KB with a tile to themselves
                                   (196, 70, 3), (196, 82, 2), (100, 100, 2), (36, 128, 3),
                                   # whole samples in registers: the forms of the kernel
                                   (100, 33, 3), (36, 256, 3), (400, 40, 2), (784, 40, 2), (196, 200, 2), (196, 320, 1),
                                   # column tiles over planes that are not whole 32-byte pieces
                                   (676, 100, 1), (900, 65, 2),
                                   # column tiles in registers
                                   (128, 33, 3), (132, 512, 2), (900, 300, 1), (400, 200, 2), (2048, 257, 1), (4096, 64, 1),
                                   # planes that are not whole 16-byte groups through the 16-byte kernels
                                   (1001, 19, 2), (2049, 2, 3), (4225, 21, 1), (129, 33, 3), (1031, 300, 1), (49, 300, 3), (17, 129, 5), (196, 600, 2), (901, 700, 1)])
def test_fused_softmax_nd_nll_equals_the_two_launches(oracle, P, C, N):
    g = np.random.default_rng(P + C)
    n = P * C * N
    x = g.standard_normal(n).astype(F32)
    lab = g.integers(0, C, P * N).astype(np.uint32)
    lab[g.random(P * N) < 0.1] = 255 if C < 255 else 0xFFFFFFFF
    for offset in (0, 1):
        p1, nll1 = empty(n, offset=offset), empty(P * N, offset=offset)
        call("anode_gpu_softmax_nd_packed_f32", P, C, N, dev(x, offset), p1)
        call("anode_gpu_softmax_nd_cat_nll_packed_f32", P, C, N, p1, dev(lab, offset), nll1)
        p2, nll2 = empty(n, offset=offset), empty(P * N, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_fused_packed_f32", P, C, N, dev(x, offset), dev(lab, offset), p2, nll2)
        assert_bit_exact(host(p2), host(p1), "fused softmax")
        assert_bit_exact(host(nll2), host(nll1), "fused nll")
        assert_close(host(p2), oracle.softmax_nd(P, C, N, x, f64=True), "fused softmax vs fp64", abs_floor=1e-30)
        # forward and backward in one launch: the bits of the three launches
        dy = g.standard_normal(P * N).astype(F32)
        dx1 = empty(n, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dev(dy, offset), p1, dev(lab, offset), dx1)
        p3, nll3, dx3 = empty(n, offset=offset), empty(P * N, offset=offset), empty(n, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32", P, C, N, dev(x, offset), dev(lab, offset),
             dev(dy, offset), p3, nll3, dx3)
        assert_bit_exact(host(p3), host(p1), "fwd+bwd fused softmax")
        assert_bit_exact(host(nll3), host(nll1), "fwd+bwd fused nll")
        assert_bit_exact(host(dx3), host(dx1), "fwd+bwd fused dx")
        assert_bit_exact(host(dx3), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, host(p1), lab), "fwd+bwd fused dx vs oracle")


ROW_FUSED_SHAPES = [(1, 5), (2, 7), (10, 32), (19, 513), (32, 600), (33, 9), (64, 300), (65, 3), (100, 17), (256, 5),
                    (40, 700), (130, 77), (208, 70), (209, 70), (212, 40), (36, 300), (92, 64), (180, 41), (225, 33), (240, 9),
                    (250, 21), (256, 33), (1012, 19), (2052, 11), (4100, 9),
                    (1000, 256), (1024, 3), (1025, 2), (2048, 2), (2049, 3), (4097, 2), (16385, 1), (40000, 1),
                    (9216, 2), (9220, 2), (12289, 2), (20000, 3), (32768, 2), (32772, 2), (50257, 2), (65540, 3),
                    (32772, 1100)]   # several rows per workgroup of the streaming kernel


@pytest.mark.parametrize("K,R", ROW_FUSED_SHAPES)
def test_fused_softmax_nll_rows_equals_the_two_launches(oracle, K, R):
    # every row kernel (thread per row, lane group, wave, workgroup in registers, workgroup streamed)
    g = np.random.default_rng(K * 3 + R)
    x = (2 * g.standard_normal(K * R)).astype(F32)
    lab = g.integers(0, K, R).astype(np.uint32)
    if R > 4:
        lab[1], lab[3] = K, 0xFFFFFFFF     # out of range: NaN
        lab[2], lab[4] = 0, K - 1          # first and last class
    for offset in (0, 1):
        p1, nll1 = empty(K * R, offset=offset), empty(R, offset=offset)
        call("anode_gpu_softmax_packed_deterministic_f32", K, R, dev(x, offset), p1)
        call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p1, dev(lab, offset), nll1)
        p2, nll2 = empty(K * R, offset=offset), empty(R, offset=offset)
        call("anode_gpu_softmax_cat_nll_fused_packed_f32", K, R, dev(x, offset), dev(lab, offset), p2, nll2)
        assert_bit_exact(host(p2), host(p1), f"fused row softmax K={K}")
        assert_bit_exact(host(nll2), host(nll1), f"fused row nll K={K}")
        assert np.array_equal(np.isnan(host(nll2)), lab >= K)
        assert_close(host(nll2), oracle.softmax_cat_nll(K, R, host(p2), lab, f64=True), "fused nll vs fp64", abs_floor=1e-6)
        # forward and backward in one launch
        dy = g.standard_normal(R).astype(F32)
        dx1 = empty(K * R, offset=offset)
        call("anode_gpu_softmax_cat_nll_bwd_packed_f32", K, R, dev(dy, offset), p1, dev(lab, offset), dx1)
        p4, nll4, dx4 = empty(K * R, offset=offset), empty(R, offset=offset), empty(K * R, offset=offset)
        call("anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32", K, R, dev(x, offset), dev(lab, offset), dev(dy, offset),
             p4, nll4, dx4)
        assert_bit_exact(host(p4), host(p1), "fwd+bwd fused softmax")
        assert_bit_exact(host(nll4), host(nll1), "fwd+bwd fused nll")
        assert_bit_exact(host(dx4), host(dx1), "fwd+bwd fused dx")
        # the channel-axis entry point with one pixel per sample is the same thing
        p3, nll3 = empty(K * R, offset=offset), empty(R, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_fused_packed_f32", 1, K, R, dev(x, offset), dev(lab, offset), p3, nll3)
        assert_bit_exact(host(p3), host(p1), "n-d fused with prefix 1")
        assert_bit_exact(host(nll3), host(nll1), "n-d fused nll with prefix 1")


def test_ref_fused_softmax_nll_known_answers():
    # the reference's known answers (tests/test_gpu.rs:615-690) through the fused entry point
    import math
    p, nll = empty(64), empty(2)
    call("anode_gpu_softmax_cat_nll_fused_packed_f32", 32, 2, dev(np.zeros(64, F32)), dev(np.array([12, 17], np.uint32)), p, nll)
    assert np.all(host(p) == F32(1.0) / F32(32.0))
    assert_close(host(nll), [math.log(32.0)] * 2, "nll", rel=1e-6)
    call("anode_gpu_softmax_cat_nll_fused_packed_f32", 32, 2, dev(np.zeros(64, F32)), dev(np.array([12, 42], np.uint32)), p, nll)
    h = host(nll)
    assert np.isfinite(h[0]) and np.isnan(h[1]) and np.isnan(h.sum())


def test_running_statistics_in_the_statistics_launch_known_answers():
    # x == 3 everywhere: mean 3, variance 0 + eps; from running values 1 and 1 at rate 1/4 (the arithmetic of
    # tests/test_gpu.rs:561-593): 1 + (3 - 1)/4 = 1.5 and 1 + (eps - 1)/4; null running arrays are skipped
    S, C, N = 49, 8, 4
    x = dev(np.full(S * C * N, 3.0, F32))
    m, v, rm, rv = empty(C), empty(C), dev(np.ones(C, F32)), dev(np.ones(C, F32))
    call("anode_gpu_batch_mean_var_online_3d1_packed_f32", S, C, N, 0.5, 0.25, x, m, v, rm, rv)
    assert np.all(host(m) == F32(3.0)) and np.all(host(v) == F32(0.5))
    assert np.all(host(rm) == F32(1.5)) and np.all(host(rv) == F32(0.875))
    m2, v2 = empty(C), empty(C)
    call("anode_gpu_batch_mean_var_online_3d1_packed_f32", S, C, N, 0.5, 0.25, x, m2, v2, None, None)
    assert np.all(host(m2) == F32(3.0)) and np.all(host(v2) == F32(0.5))


def test_ref_online_average_quarter_steps(oracle):
    # tests/test_gpu.rs:561-593: y0 = 0, x = 1, rate .25 -> 0.25 then 0.4375, exactly
    y = dev(np.zeros(1024, F32))
    x = dev(np.ones(1024, F32))
    call("anode_gpu_online_average_packed_f32", 1024, 0.25, x, y)
    assert np.all(host(y) == F32(0.25))
    call("anode_gpu_online_average_packed_f32", 1024, 0.25, x, y)
    assert np.all(host(y) == F32(0.4375))
    g = np.random.default_rng(2)
    a, b = g.standard_normal(3001).astype(F32), g.standard_normal(3001).astype(F32)
    yb = dev(b, 1)
    call("anode_gpu_online_average_packed_f32", 3001, 0.1, dev(a, 1), yb)
    assert_bit_exact(host(yb), oracle.online_average(0.1, a, b), "online average")


def test_arg_max_rows(oracle):
    g = np.random.default_rng(3)
    for K, R in [(10, 32), (1000, 256), (1, 5), (64, 7), (65, 3), (5000, 2), (1001, 33), (8, 1000), (4096, 9),
                 # rows that start at every distance from a 128-byte line (K = 4 * odd), few and many passes per row
                 (12, 40), (20, 33), (100, 64), (204, 20), (1012, 17), (2044, 9), (260, 70)]:
        # a coarse grid of values: ties within a lane's group of four, across lanes and across loop passes
        x = ((g.integers(-3, 4, K * R) * 0.5).astype(F32) if K in (8, 1001, 4096, 12, 100, 1012, 260)
             else g.standard_normal(K * R).astype(F32))
        xr = x.reshape(R, K)
        if R > 3 and K > 4:
            xr[0, :] = 1.0                       # all equal: first index
            xr[1, :] = -np.inf                   # nothing exceeds -inf: 0
            xr[2, 0] = np.nan
            xr[2, 3] = np.nan                    # NaN never wins
            xr[3, K - 1] = xr[3, K - 2] = 9.0    # tie: the first of the two
        for offset in (0, 1):  # aligned rows take the 16-byte path when K is a multiple of 4
            out = empty(R, dtype=torch.int32)
            call("anode_gpu_arg_max_packed_u32", K, R, dev(x, offset), out)
            assert_bit_exact(host(out).view(np.uint32), oracle.arg_max_rows(K, R, x), f"arg_max K={K} offset={offset}")
