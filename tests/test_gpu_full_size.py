"""GPU parity at the full sizes of BASELINE.json's configs: per-channel and
bit-exact results against the (multi-threaded) oracle, large element-wise
results through slices against the oracle plus size-independent properties
(normalised output has zero mean / unit variance, the BN input gradient is
orthogonal to 1 and to the normalised output, softmax rows sum to one,
dequantize then quantise-back is the identity on codes)."""
import numpy as np
import pytest
import torch

from gpu_util import F32, assert_bit_exact, assert_close, call, dev, empty, host, rms

pytestmark = pytest.mark.gpu


def normal(n, seed, mean=0.0, std=1.0):
    g = np.random.default_rng(seed)
    x = g.standard_normal(n, dtype=np.float32)
    if std != 1.0:
        x *= F32(std)
    if mean != 0.0:
        x += F32(mean)
    return x


def test_config1_u8_image_batch_cast_and_dequantize(oracle):
    n = 256 * 3 * 224 * 224
    q = np.random.default_rng(0).integers(0, 256, n, dtype=np.uint8)
    qd = dev(q)
    y = empty(n)
    call("anode_gpu_dequantize_u8_packed_f32", n, 0.0, 1.0, qd, y)
    yh = host(y)
    assert_bit_exact(yh, oracle.dequantize_u8(0.0, 1.0, q), "dequantize 38.5M")
    # round trip: rounding y*255 recovers the code
    assert np.array_equal(np.rint(yh.astype(np.float64) * 255).astype(np.uint8), q)
    u = empty(n, dtype=torch.int32)
    call("anode_gpu_upcast_u8_packed_u32", n, qd, u)
    assert_bit_exact(host(u).view(np.uint32), oracle.upcast_u8(q), "upcast 38.5M")


def test_config1_additive_full_size(oracle):
    """What config 1 words beyond the reference's two casts, at [256,3,224,224]: u8 -> f32 with per-channel
    ImageNet normalisation in one pass, and an N(0,1) f32 tensor quantised to u8 (scale 8/255, zero point at -4,
    round-half-even).  Bit-exact against the oracle; the quantiser has no counterpart in the reference."""
    n_img, C, S = 256, 3, 224 * 224
    n = n_img * C * S
    g = np.random.default_rng(1)
    q = g.integers(0, 256, n, dtype=np.uint8)
    mean = np.array([0.485, 0.456, 0.406], F32)
    std = np.array([0.229, 0.224, 0.225], F32)
    a = (F32(1.0) / (F32(255.0) * std)).astype(F32)
    b = (-mean / std).astype(F32)
    y = empty(n)
    call("anode_gpu_bcast_dequantize_u8_I1b_I2abc_Oabc_packed_f32", S, C, n_img, dev(a), dev(b), dev(q), y)
    yh = host(y)
    assert_bit_exact(yh, oracle.bcast_dequantize_u8(S, C, n_img, a, b, q), "per-channel dequantize 38.5M")
    # size-independent: undoing the affine per channel recovers every code
    ch = np.tile(np.repeat(np.arange(C), S), n_img)
    back = np.rint((yh.astype(np.float64) - b.astype(np.float64)[ch]) / a.astype(np.float64)[ch])
    assert np.array_equal(back.astype(np.uint8), q)
    del yh, back, ch

    z = g.standard_normal(n, dtype=np.float32)
    zq = empty(n, dtype=torch.uint8)
    call("anode_gpu_quantize_u8_packed_f32", n, -4.0, 4.0, dev(z), zq)
    zh = host(zq)
    assert_bit_exact(zh, oracle.quantize_u8(-4.0, 4.0, z), "quantize 38.5M")
    # dequantising the codes lands within half a step of the clamped input, and quantising again is the identity
    deq = empty(n)
    call("anode_gpu_dequantize_u8_packed_f32", n, -4.0, 4.0, zq, deq)
    step = 8.0 / 255.0
    assert float(np.max(np.abs(host(deq).astype(np.float64) - np.clip(z, -4, 4)))) <= 0.5 * step + 2e-6   # (fp32 rounding of x - lo and of the dequantised value)
    zq2 = empty(n, dtype=torch.uint8)
    call("anode_gpu_quantize_u8_packed_f32", n, -4.0, 4.0, deq, zq2)
    assert np.array_equal(host(zq2), zh)


def _bn_full(oracle, S, C, N, seed, mean_shift, std, slice_samples):
    """BN forward + backward launch set at full size."""
    eps = 1e-5
    n = S * C * N
    x = normal(n, seed, mean_shift, std)
    dy = normal(n, seed + 1)
    xd, dyd = dev(x), dev(dy)
    dims = (S, C, N)
    mean_d, var_d = empty(C), empty(C)
    call("anode_gpu_batch_mean_3d1_packed_f32", *dims, xd, mean_d)
    call("anode_gpu_batch_var_3d1_packed_f32", *dims, eps, xd, mean_d, var_d)
    mean, var = host(mean_d), host(var_d)
    assert_close(mean, oracle.batch_mean(*dims, x, f64=True), "mean")
    assert_close(var, oracle.batch_var(*dims, eps, x, mean, f64=True), "var")

    y_d = empty(n)
    call("anode_gpu_batch_norm_3d1_packed_f32", *dims, xd, mean_d, var_d, y_d)
    dmean_d, dvar_d, dx_d = empty(C), empty(C), empty(n)
    call("anode_gpu_batch_norm_bwd_3d1_packed_f32", *dims, dyd, var_d, dx_d)
    call("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", *dims, dyd, var_d, dmean_d)
    call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", *dims, dyd, xd, mean_d, var_d, dvar_d)
    dmean1, dvar = host(dmean_d).copy(), host(dvar_d).copy()
    ref = oracle.batch_norm_bwd_mean(*dims, dy, var, f64=True)
    assert_close(dmean1, ref, "norm_bwd_mean", abs_floor=1e-6 * rms(ref))
    ref = oracle.batch_norm_bwd_var(*dims, dy, x, mean, var, f64=True)
    assert_close(dvar, ref, "norm_bwd_var", abs_floor=1e-6 * rms(ref))
    call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *dims, dvar_d, xd, mean_d, dx_d)
    call("anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", *dims, dvar_d, xd, mean_d, dmean_d)
    dmean = host(dmean_d).copy()
    assert_close(dmean, oracle.batch_var_bwd_mean(*dims, dvar, x, mean, dmean_in=dmean1, f64=True), "var_bwd_mean acc",
                 abs_floor=1e-10)
    call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", *dims, dmean_d, dx_d)

    # element-wise outputs: the first and last samples against the oracle (same per-channel inputs)
    y, dx = host(y_d), host(dx_d)
    CS = C * S
    for lo, hi in slice_samples:
        sl = slice(lo * CS, hi * CS)
        sub = (S, C, hi - lo)
        assert_bit_exact(y[sl], oracle.batch_norm(*sub, x[sl], mean, var), f"y samples {lo}:{hi}")
        d = oracle.batch_norm_bwd(*sub, dy[sl], var)
        # var_bwd and mean_bwd divide by the FULL batch count: restate with the full n
        nf = F32(S) * F32(N)
        ch = np.tile(np.repeat(np.arange(C), S), hi - lo)
        d = d + (dvar[ch] * (x[sl] - mean[ch]) * F32(2.0) / nf)
        d = d + dmean[ch] / nf
        assert_bit_exact(dx[sl], d.astype(F32), f"dx samples {lo}:{hi}")

    # size-independent properties over the whole array (fp64 on the device)
    yt = y_d.view(N, C, S).double()
    dxt = dx_d.view(N, C, S).double()
    m = yt.mean((0, 2)).cpu().numpy()
    v = yt.var((0, 2), unbiased=False).cpu().numpy()
    assert np.all(np.abs(m) < 1e-5)
    assert_close(v, 1 - eps / var.astype(np.float64), "var of y", rel=1e-4)
    dyt = dyd.view(N, C, S).double()
    scale = dyt.abs().sum((0, 2)).cpu().numpy() / np.sqrt(var.astype(np.float64))  # sum |dy| * rs per channel
    assert np.all(np.abs(dxt.sum((0, 2)).cpu().numpy()) <= 1e-5 * scale)          # sum dx = 0
    assert np.all(np.abs((dxt * yt).sum((0, 2)).cpu().numpy()) <= 3e-5 * scale)   # sum dx * y_hat = 0


def test_config2a_batch_norm_256x64x112x112(oracle):
    _bn_full(oracle, 112 * 112, 64, 256, seed=20, mean_shift=2.0, std=3.0, slice_samples=[(0, 2), (254, 256)])


def test_config2b_batch_norm_256x2048x7x7(oracle):
    _bn_full(oracle, 49, 2048, 256, seed=30, mean_shift=2.0, std=3.0, slice_samples=[(0, 256)])


def test_config4_batch_norm_3d_with_relu(oracle):
    S, C, N = 128 * 128 * 128, 32, 2
    _bn_full(oracle, S, C, N, seed=40, mean_shift=0.0, std=1.0, slice_samples=[(0, 1), (1, 2)])
    n = S * C * N
    x = normal(n, 41)
    dy = normal(n, 42)
    xd = dev(x)
    call("anode_gpu_positive_clip_flat_map_f32", n, xd, xd)              # in place, bench_unet3d.rs:103
    yh = host(xd)
    assert_bit_exact(yh, oracle.flat_map("positive_clip", x), "relu 134M")
    dx = empty(n)
    call("anode_gpu_positive_clip_flat_map_bwd_f32", n, dev(dy), xd, dx)
    assert_bit_exact(host(dx), oracle.flat_map2("positive_clip_bwd", dy, yh), "relu bwd 134M")
    call("anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32", n, dev(dy), xd, dx)
    assert_bit_exact(host(dx), oracle.flat_map2("copy_unit_step_join", dy, yh), "relu mask join 134M")


def test_config3a_softmax_256x1000(oracle):
    K, R = 1000, 256
    g = np.random.default_rng(50)
    x = (2 * g.standard_normal(K * R)).astype(F32)  # N(0, 4): sigma = 2
    lab = g.integers(0, K, R).astype(np.uint32)
    for name in ("anode_gpu_softmax_packed_block_f32", "anode_gpu_softmax_packed_deterministic_f32"):
        p_d = empty(K * R)
        call(name, K, R, dev(x), p_d)
        p = host(p_d)
        assert_close(p, oracle.softmax(K, R, x, f64=True), name, abs_floor=1e-30)
    nll = empty(R)
    call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p_d, dev(lab), nll)
    assert_close(host(nll), oracle.softmax_cat_nll(K, R, p, lab, f64=True), "nll", abs_floor=1e-6)
    dx = empty(K * R)
    call("anode_gpu_softmax_cat_nll_bwd_packed_f32", K, R, dev(np.ones(R, F32)), p_d, dev(lab), dx)
    assert_bit_exact(host(dx), oracle.softmax_cat_nll_bwd(K, R, np.ones(R, F32), p, lab), "nll bwd")


def test_config3b_softmax_nd_8x19x512x1024(oracle):
    P, C, N = 512 * 1024, 19, 8
    n = P * C * N
    g = np.random.default_rng(60)
    x = g.standard_normal(n, dtype=np.float32)
    lab = g.integers(0, C, P * N).astype(np.uint32)
    lab[g.random(P * N) < 0.05] = 255   # 5 % ignore-index: NaN nll, unmasked gradient (the reference has no mask)
    p_d = empty(n)
    call("anode_gpu_softmax_nd_packed_f32", P, C, N, dev(x), p_d)
    p = host(p_d)
    assert_close(p, oracle.softmax_nd(P, C, N, x, f64=True), "softmax_nd 80M", abs_floor=1e-30)
    sums = p_d.view(N, C, P).double().sum(1)
    assert float((sums - 1).abs().max()) < 1e-5
    nll = empty(P * N)
    call("anode_gpu_softmax_nd_cat_nll_packed_f32", P, C, N, p_d, dev(lab), nll)
    nh = host(nll)
    assert np.array_equal(np.isnan(nh), lab == 255)
    assert_close(nh, oracle.softmax_nd_cat_nll(P, C, N, p, lab, f64=True), "nd nll", abs_floor=1e-6)
    dy = np.ones(P * N, F32)            # the adjoint of a batch sum
    dx = empty(n)
    call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dev(dy), p_d, dev(lab), dx)
    assert_bit_exact(host(dx), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy, p, lab), "nd nll bwd 80M")
