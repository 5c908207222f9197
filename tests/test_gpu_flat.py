"""GPU parity: flat maps, the flat join, u8 widening (upcast, dequantize),
one-hot and the smooth F1 loss, through the C ABI against the oracle."""
import numpy as np
import pytest

from gpu_util import F32, assert_bit_exact, assert_close, call, dev, empty, host, rms

import torch

pytestmark = pytest.mark.gpu

SPECIALS = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.5, -2.25, 1e38, -1e38,
                     1.1754944e-38, -1.1754944e-38, 88.0, -88.0, 104.0, -104.0, 0.5, -0.5], F32)

LENGTHS = [1, 2, 3, 4, 5, 15, 16, 17, 63, 64, 255, 1024, 1027, 4095, 4096, 4111, 4096 * 3 + 1, 1 << 20, (1 << 20) + 3]

# entry point -> (oracle map name, bit-exact against the fp32 restatement?)
MAPS = {
    "anode_gpu_copy_flat_map_f32": ("copy", True),
    "anode_gpu_modulus_flat_map_f32": ("modulus", True),
    "anode_gpu_square_flat_map_f32": ("square", True),
    "anode_gpu_sqrt_flat_map_f32": ("sqrt", True),          # correctly rounded on both sides
    "anode_gpu_positive_clip_flat_map_f32": ("positive_clip", True),
    "anode_gpu_unit_step_flat_map_f32": ("unit_step", True),
    "anode_gpu_logistic_flat_map_f32": ("logistic", False),  # libm-dependent: tolerance class
    "anode_gpu_normal_cdf_flat_map_f32": ("normal_cdf", False),
    "anode_gpu_tanh_flat_map_f32": ("tanh", False),
    "anode_gpu_rcosh2_flat_map_f32": ("rcosh2", False),
    # whitelisted by the reference's build.rs:101-102, defined only here (functors: flat_map.cu:242-278)
    "anode_gpu_log_positive_clip_flat_map_f32": ("log_positive_clip", False),
    "anode_gpu_positive_reciprocal_flat_map_f32": ("positive_reciprocal", True),  # one correctly rounded division
}


def data(n, seed):
    g = np.random.default_rng(seed)
    x = (3 * g.standard_normal(n)).astype(F32)
    k = min(n, SPECIALS.size)
    x[:k] = SPECIALS[:k]
    return x


@pytest.mark.parametrize("name", sorted(MAPS))
def test_flat_maps(oracle, name):
    op, exact = MAPS[name]
    for n in LENGTHS:
        for offset in (0, 1):
            x = data(n, n)
            if op == "sqrt":
                x = np.where(np.isnan(x), x, np.abs(x)).astype(F32)
            y = empty(n, offset=offset)
            call(name, n, dev(x, offset), y)
            got = host(y)
            if exact:
                assert_bit_exact(got, oracle.flat_map(op, x), f"{op} n={n} offset={offset}")
            else:
                with np.errstate(all="ignore"):
                    ref = oracle.flat_map(op, x, f64=True)
                # results that underflow fp32 (rcosh2, logistic tails) are held to an absolute floor;
                # 0.5*(1+erf) cancels in fp32 for negative x by the reference's own formula: one ulp of 1
                floor = 2e-7 if op == "normal_cdf" else 1e-37
                assert_close(got, ref, f"{op} n={n} offset={offset}", rel=1e-5, abs_floor=floor)


def test_positive_clip_in_place_and_sign_rules(oracle):
    # src/ops_gpu.rs:7912-7918: called with y == x
    n = 100003
    x = data(n, 1)
    buf = dev(x)
    call("anode_gpu_positive_clip_flat_map_f32", n, buf, buf)
    got = host(buf)
    assert_bit_exact(got, oracle.flat_map("positive_clip", x), "in-place relu")
    i = list(SPECIALS).index(F32(-2.25))
    assert got[i] == 0 and np.signbit(got[i])          # x * 0.0 keeps the sign: -0.0
    assert np.isnan(got[list(SPECIALS).index(F32(-np.inf))])  # -inf * 0 = NaN, as the reference


def test_two_input_maps_and_in_place_backward(oracle):
    for n in (5, 1027, (1 << 20) + 1):
        a, b = data(n, 2), data(n, 3)[::-1].copy()
        for name, op in [("anode_gpu_positive_clip_flat_map_bwd_f32", "positive_clip_bwd"),
                         ("anode_gpu_logistic_flat_map_bwd_f32", "logistic_bwd"),
                         ("anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32", "copy_unit_step_join")]:
            for offset in (0, 1):
                out = empty(n, offset=offset)
                call(name, n, dev(a, offset), dev(b, offset), out)
                with np.errstate(all="ignore"):
                    assert_bit_exact(host(out), oracle.flat_map2(op, a, b), f"{op} n={n}")
        # src/ops_gpu.rs:7931-7937: ReLU backward called with dx == dy
        buf = dev(a)
        call("anode_gpu_positive_clip_flat_map_bwd_f32", n, buf, dev(b), buf)
        with np.errstate(all="ignore"):
            assert_bit_exact(host(buf), oracle.flat_map2("positive_clip_bwd", a, b), "in-place relu bwd")


def test_maps_with_arrays_that_lie_differently(oracle):
    # one- and two-input maps with every array at its own element offset, guard bands round the output
    import torch
    for n in (7, 1027, 300001):
        a, b = data(n, 6), data(n, 7)[::-1].copy()
        for off_a, off_b, off_out in [(0, 0, 1), (1, 0, 0), (0, 3, 0), (1, 2, 3), (2, 2, 0)]:
            for name, op, two in [("anode_gpu_positive_clip_flat_map_bwd_f32", "positive_clip_bwd", True),
                                  ("anode_gpu_M1_copy_map_M2_unit_step_map_R_product_reduce_flat_join_f32",
                                   "copy_unit_step_join", True),
                                  ("anode_gpu_square_flat_map_f32", "square", False)]:
                buf = torch.full((n + 40,), 9191.0, dtype=torch.float32, device="cuda")
                out = buf[16 + off_out:16 + off_out + n]
                if two:
                    call(name, n, dev(a, off_a), dev(b, off_b), out)
                    want = oracle.flat_map2(op, a, b)
                else:
                    call(name, n, dev(a, off_a), out)
                    want = oracle.flat_map(op, a)
                h = host(buf)
                assert np.all(h[:16 + off_out] == 9191.0) and np.all(h[16 + off_out + n:] == 9191.0), (name, n)
                with np.errstate(all="ignore"):
                    assert_bit_exact(h[16 + off_out:16 + off_out + n], want, f"{op} n={n} offsets {off_a} {off_b} {off_out}")


@pytest.mark.parametrize("c", [0.01, 0.0, -0.5, 2.0])
def test_leaky_relu(oracle, c):
    n = 70001
    x, dy = data(n, 4), data(n, 5)[::-1].copy()
    y = empty(n)
    call("anode_gpu_leaky_relu_flat_map_f32", n, c, dev(x), y)
    with np.errstate(all="ignore"):
        assert_bit_exact(host(y), oracle.flat_map("leaky_relu", x, c=c), "leaky relu")
        dx = empty(n)
        call("anode_gpu_leaky_relu_flat_map_bwd_f32", n, c, dev(dy), y, dx)
        assert_bit_exact(host(dx), oracle.flat_map2("leaky_relu_bwd", dy, host(y), c=c), "leaky relu bwd")


# ---- u8 widening -------------------------------------------------------------

def test_ref_dequantize_ones_is_exactly_one_over_255():
    # tests/test_gpu.rs:738-758
    n = 32 * 32 * 3
    y = empty(n)
    call("anode_gpu_dequantize_u8_packed_f32", n, 0.0, 1.0, dev(np.ones(n, np.uint8)), y)
    assert np.all(host(y) == F32(1.0) / F32(255.0))


@pytest.mark.parametrize("lo,hi", [(0.0, 1.0), (-1.0, 1.0), (0.1, 0.7), (-123.456, 789.01)])
def test_dequantize_all_codes_and_ragged_lengths(oracle, lo, hi):
    codes = np.arange(256, dtype=np.uint8)
    y = empty(256)
    call("anode_gpu_dequantize_u8_packed_f32", 256, lo, hi, dev(codes), y)
    assert_bit_exact(host(y), oracle.dequantize_u8(lo, hi, codes), "all 256 codes")
    g = np.random.default_rng(0)
    for n in LENGTHS:
        q = g.integers(0, 256, n, dtype=np.uint8)
        for off_in, off_out in [(0, 0), (1, 0), (0, 1), (3, 2), (4, 4)]:
            y = empty(n, offset=off_out)
            call("anode_gpu_dequantize_u8_packed_f32", n, lo, hi, dev(q, off_in), y)
            assert_bit_exact(host(y), oracle.dequantize_u8(lo, hi, q), f"n={n} offsets=({off_in},{off_out})")


def test_upcast(oracle):
    g = np.random.default_rng(1)
    for n in LENGTHS:
        q = g.integers(0, 256, n, dtype=np.uint8)
        if n >= 256:
            q[:256] = np.arange(256)
        for off_in, off_out in [(0, 0), (1, 0), (0, 1), (2, 3)]:
            y = empty(n, dtype=torch.int32, offset=off_out)
            call("anode_gpu_upcast_u8_packed_u32", n, dev(q, off_in), y)
            assert_bit_exact(host(y).view(np.uint32), oracle.upcast_u8(q), f"upcast n={n}")


# ---- one-hot -------------------------------------------------------------------

@pytest.mark.parametrize("d0,K,d2", [(1, 4, 7), (5, 3, 2), (64, 19, 3), (100, 1, 2), (7, 10, 5), (4096, 5, 2), (12, 40, 3),
                                     # the flat walk (planes of whole 16-byte groups from 16 pixels on, any plane from 512
                                     # on): its shortest planes and the next shorter ones, groups across the end of a
                                     # plane, of a sample and of the array, one class
                                     (16, 3, 5), (20, 7, 3), (512, 3, 2), (513, 5, 3), (511, 5, 3), (515, 3, 1), (517, 1, 3),
                                     (1025, 19, 2), (4225, 2, 1)])
def test_one_hot(oracle, d0, K, d2):
    g = np.random.default_rng(d0 + K)
    lab = g.integers(0, K + 2, d0 * d2).astype(np.uint32)  # some labels have no class: all-zero column
    for offset in (0, 1):
        y = empty(d0 * K * d2, offset=offset)
        call("anode_gpu_discrete_one_hot_3d1_packed_f32", d0, K, d2, dev(lab, offset), y)
        assert_bit_exact(host(y), oracle.one_hot(d0, K, d2, lab), f"one_hot offset={offset}")


# ---- smooth F1 -----------------------------------------------------------------

@pytest.mark.parametrize("d0,K,d2", [(50, 3, 2), (1, 5, 4), (4096, 2, 2), (5000, 3, 1), (70000, 2, 2), (333, 17, 3)])
def test_f1_loss_and_bwd(oracle, d0, K, d2):
    g = np.random.default_rng(d0)
    n = d0 * K * d2
    x = g.random(n).astype(F32)
    t = (g.random(n) > 0.5).astype(F32)
    dy = g.standard_normal(K * d2).astype(F32)
    eps = 1e-3
    for offset in (0, 1):
        y = empty(K * d2, offset=offset)
        call("anode_gpu_smooth_negative_f1_loss_3d1_packed_f32", d0, K, d2, eps, dev(x, offset), dev(t, offset), y)
        assert_close(host(y), oracle.f1_loss(d0, K, d2, eps, x, t, f64=True), "f1 loss")
        dx = empty(n, offset=offset)
        call("anode_gpu_smooth_negative_f1_loss_3d1_bwd_packed_f32", d0, K, d2, eps, dev(dy, offset), dev(x, offset),
             dev(t, offset), dx)
        ref = oracle.f1_loss_bwd(d0, K, d2, eps, dy, x, t, f64=True)
        assert_close(host(dx), ref, "f1 loss bwd", abs_floor=1e-6 * rms(ref))
        assert_bit_exact(host(dx), oracle.f1_loss_bwd(d0, K, d2, eps, dy, x, t), "f1 loss bwd vs fp32")
