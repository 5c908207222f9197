"""GPU parity of the entry points around the path: the gpudevicemem neighbours (fills, add/mult, scalar broadcast,
batch sum, per-sample division, running-statistics add) and the "ignore" variants of the NLL kernels.

None of these is pinned by a reference kernel (gpudevicemem's source is not part of the reference tree, and the
reference has no ignore-index): elementwise ones are single IEEE operations and are compared bit for bit with numpy
fp32 / the oracle's fmaf; the sum is compared with the fp64 sum at 1e-5; the values the reference's tests assert at
this boundary (fills, tests/test_gpu.rs:245-290; the sum-join value 10.0, :302-353) are checked exactly.
"""
import numpy as np
import pytest

from gpu_util import F32, assert_bit_exact, assert_close, call, dev, empty, host
from oracle import binding as oracle

pytestmark = pytest.mark.gpu

LENS = [1, 3, 4, 255, 1024, 4099, 1 << 20]


@pytest.mark.parametrize("n", LENS)
def test_fill_add_mult_nonzero(n):
    g = np.random.default_rng(n)
    x = g.standard_normal(n).astype(F32)
    x[:: 5] = 0.0
    if n > 3:
        x[1], x[2], x[3] = -0.0, np.inf, np.nan
    y0 = g.standard_normal(n).astype(F32)
    for offset in (0, 1):
        y = empty(n, offset=offset)
        call("anode_gpu_set_constant_packed_f32", n, 0.0, y)
        assert_bit_exact(host(y), np.zeros(n, F32), "set_zeros")
        call("anode_gpu_set_constant_packed_f32", n, 1.0, y)
        assert_bit_exact(host(y), np.ones(n, F32), "set_constant 1")
        call("anode_gpu_set_constant_packed_f32", n, -2.5, y)
        assert_bit_exact(host(y), np.full(n, -2.5, F32), "set_constant")

        y = dev(y0, offset)
        call("anode_gpu_add_packed_f32", n, dev(x, offset), y)
        with np.errstate(all="ignore"):
            assert_bit_exact(host(y), y0 + x, "add")
        y = dev(y0, offset)
        call("anode_gpu_mult_packed_f32", n, dev(x, offset), y)
        with np.errstate(all="ignore"):
            assert_bit_exact(host(y), y0 * x, "mult")
        y = empty(n, offset=offset)
        call("anode_gpu_is_nonzero_packed_f32", n, dev(x, offset), y)
        assert_bit_exact(host(y), (x != 0).astype(F32), "is_nonzero")
        y = dev(y0, offset)
        call("anode_gpu_online_add_packed_f32", n, 0.1, dev(x, offset), y)
        with np.errstate(all="ignore"):
            assert_bit_exact(host(y), oracle.online_add(0.1, x, y0), "online_add")
        y = dev(y0, offset)
        call("anode_gpu_online_discount_packed_f32", n, 0.9, dev(x, offset), y)
        with np.errstate(all="ignore"):
            assert_bit_exact(host(y), oracle.online_discount(0.9, x, y0), "online_discount")


@pytest.mark.parametrize("n", LENS)
def test_bcast_scalar(n):
    s = np.array([1.625], F32)
    y0 = np.random.default_rng(n).standard_normal(n).astype(F32)
    for offset in (0, 1):
        y = empty(n, offset=offset)
        call("anode_gpu_bcast_packed_f32", n, dev(s), y)
        assert_bit_exact(host(y), np.full(n, s[0], F32), "bcast")
        y = dev(y0, offset)
        call("anode_gpu_bcast_packed_accumulate_f32", n, dev(s), y)
        assert_bit_exact(host(y), y0 + s[0], "bcast accumulate")


@pytest.mark.parametrize("n", LENS + [10, 5_000_000])
def test_sum_packed(n):
    g = np.random.default_rng(n)
    x = (1 + g.standard_normal(n)).astype(F32)
    for offset in (0, 1):
        y = dev(np.array([7.0], F32))
        call("anode_gpu_sum_packed_deterministic_f32", n, dev(x, offset), y)
        ref = oracle.sum_packed(x)
        assert_close(host(y), [ref], "sum", abs_floor=1e-6 * np.sqrt(n))
        first = host(y).copy()
        call("anode_gpu_sum_packed_deterministic_f32", n, dev(x, offset), y)
        assert_bit_exact(host(y), first, "sum is reproducible")
        y = dev(np.array([7.0], F32))
        call("anode_gpu_sum_packed_accumulate_deterministic_f32", n, dev(x, offset), y)
        assert_bit_exact(host(y), F32(7.0) + first, "sum accumulate")


def test_sum_join_value_of_the_reference_test():
    # tests/test_gpu.rs:302-353 sums ten arrays of ones and expects 10.0; here: the batch sum of ten ones
    y = empty(1)
    call("anode_gpu_sum_packed_deterministic_f32", 10, dev(np.ones(10, F32)), y)
    assert host(y)[0] == F32(10.0)
    call("anode_gpu_sum_packed_deterministic_f32", 0, dev(np.ones(1, F32)), y)
    assert host(y)[0] == F32(0.0)


@pytest.mark.parametrize("inner,outer", [(1, 7), (10, 32), (1000, 3), (150528, 4), (37, 1)])
def test_flat_bcast_rdiv(inner, outer):
    g = np.random.default_rng(inner + outer)
    x = g.standard_normal(inner * outer).astype(F32)
    r = (0.5 + g.random(outer)).astype(F32)
    for offset in (0, 1):
        y = empty(inner * outer, offset=offset)
        call("anode_gpu_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32", inner, outer, dev(x, offset), dev(r), y)
        assert_bit_exact(host(y), oracle.flat_bcast_rdiv(inner, outer, x, r), "rdiv")


def test_gpudevicemem_link_names(oracle=oracle):
    # the five entry points anode calls by their gpudevicemem names (src/ops_gpu.rs:7486-7505, 7595-7614, 9592-9600):
    # against the oracle / numpy, and bit for bit against the anode_gpu_* twins they forward to
    g = np.random.default_rng(11)
    n = 4099
    x = (1 + g.standard_normal(n)).astype(F32)
    y = dev(np.array([7.0], F32))
    call("gpudevicemem_sum_packed_deterministic_f32", n, dev(x), y)
    assert_close(host(y), [oracle.sum_packed(x)], "sum", abs_floor=1e-6 * np.sqrt(n))
    twin = dev(np.array([7.0], F32))
    call("anode_gpu_sum_packed_deterministic_f32", n, dev(x), twin)
    assert_bit_exact(host(y), host(twin), "sum twin")
    first = host(y).copy()
    y = dev(np.array([7.0], F32))
    call("gpudevicemem_sum_packed_accumulate_deterministic_f32", n, dev(x), y)
    assert_bit_exact(host(y), F32(7.0) + first, "sum accumulate")
    call("gpudevicemem_sum_packed_deterministic_f32", 10, dev(np.ones(10, F32)), y)
    assert host(y)[0] == F32(10.0)    # the value the reference's sum-join test expects (tests/test_gpu.rs:302-353)

    s, y0 = np.array([1.625], F32), g.standard_normal(n).astype(F32)
    y = empty(n)
    call("gpudevicemem_bcast_packed_f32", n, dev(s), y)
    assert_bit_exact(host(y), np.full(n, s[0], F32), "bcast")
    y = dev(y0)
    call("gpudevicemem_bcast_packed_accumulate_f32", n, dev(s), y)
    assert_bit_exact(host(y), y0 + s[0], "bcast accumulate")

    inner, outer = 1000, 3
    xr = g.standard_normal(inner * outer).astype(F32)
    r = (0.5 + g.random(outer)).astype(F32)
    y = empty(inner * outer)
    call("gpudevicemem_flat_bcast_rdiv_I1ab_I2b_Oab_packed_f32", inner, outer, dev(xr), dev(r), y)
    assert_bit_exact(host(y), oracle.flat_bcast_rdiv(inner, outer, xr, r), "rdiv")


@pytest.mark.parametrize("K,R", [(10, 32), (1000, 5), (1, 3), (33, 64)])
def test_row_nll_ignore(K, R):
    g = np.random.default_rng(K * R)
    p = oracle.softmax(K, R, g.standard_normal(K * R).astype(F32))
    lab = g.integers(0, K, R).astype(np.uint32)
    lab[::3] = 255 + K
    lab[1] = 0xFFFFFFFF
    dy = g.standard_normal(R).astype(F32)
    keep = lab < K
    nll = empty(R)
    call("anode_gpu_softmax_cat_nll_ignore_packed_f32", K, R, dev(p), dev(lab), nll)
    plain = empty(R)
    call("anode_gpu_softmax_cat_nll_packed_f32", K, R, dev(p), dev(lab), plain)
    want = np.where(keep, host(plain), F32(0.0)).astype(F32)
    assert_bit_exact(host(nll), want, "row nll ignore")
    assert np.all(np.isnan(host(plain)[~keep]))
    dy_masked = np.where(keep, dy, F32(0.0)).astype(F32)
    dx = empty(K * R)
    call("anode_gpu_softmax_cat_nll_bwd_ignore_packed_f32", K, R, dev(dy), dev(p), dev(lab), dx)
    assert_bit_exact(host(dx), oracle.softmax_cat_nll_bwd(K, R, dy_masked, p, lab), "row bwd ignore")
    assert np.all(host(dx).reshape(R, K)[~keep] == 0)
    old = g.standard_normal(K * R).astype(F32)
    dx = dev(old)
    call("anode_gpu_softmax_cat_nll_bwd_ignore_packed_accumulate_f32", K, R, dev(dy), dev(p), dev(lab), dx)
    assert_bit_exact(host(dx), oracle.softmax_cat_nll_bwd(K, R, dy_masked, p, lab, dx_in=old), "row bwd ignore acc")
    assert_bit_exact(host(dx).reshape(R, K)[~keep], old.reshape(R, K)[~keep], "ignored rows untouched")


@pytest.mark.parametrize("P,C,N", [(64, 19, 2), (37, 5, 3), (1, 10, 8), (4096, 19, 2), (8, 70, 2), (1025, 7, 2),
                                   (515, 3, 3)])
def test_nd_nll_ignore(P, C, N):
    g = np.random.default_rng(P * C + N)
    p = oracle.softmax_nd(P, C, N, g.standard_normal(P * C * N).astype(F32))
    lab = g.integers(0, C, P * N).astype(np.uint32)
    lab[g.random(P * N) < 0.2] = 255
    dy = g.standard_normal(P * N).astype(F32)
    keep = lab < C
    for offset in (0, 1):
        nll = empty(P * N, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_ignore_packed_f32", P, C, N, dev(p, offset), dev(lab, offset), nll)
        ref = np.where(keep, oracle.softmax_nd_cat_nll(P, C, N, p, np.where(keep, lab, 0).astype(np.uint32)), F32(0.0))
        assert_close(host(nll), ref.astype(np.float64), "nd nll ignore", abs_floor=1e-6)
        assert np.all(host(nll)[~keep] == 0)
        plain = empty(P * N, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_packed_f32", P, C, N, dev(p, offset), dev(lab, offset), plain)
        assert_bit_exact(host(nll)[keep], host(plain)[keep], "in-range pixels identical to the plain entry point")
        dy_masked = np.where(keep, dy, F32(0.0)).astype(F32)
        dx = empty(P * C * N, offset=offset)
        call("anode_gpu_softmax_nd_cat_nll_bwd_ignore_packed_f32", P, C, N, dev(dy, offset), dev(p, offset),
             dev(lab, offset), dx)
        assert_bit_exact(host(dx), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy_masked, p, lab), "nd bwd ignore")
        old = g.standard_normal(P * C * N).astype(F32)
        dx = dev(old, offset)
        call("anode_gpu_softmax_nd_cat_nll_bwd_ignore_packed_accumulate_f32", P, C, N, dev(dy, offset), dev(p, offset),
             dev(lab, offset), dx)
        assert_bit_exact(host(dx), oracle.softmax_nd_cat_nll_bwd(P, C, N, dy_masked, p, lab, dx_in=old),
                         "nd bwd ignore accumulate")


def test_momentum_step_recipe():
    # src/ops.rs:1425-1430: buffer <- momentum * buffer + grad, then params <- params + step * buffer
    buf = dev(np.zeros(1000, F32))
    grad = dev(np.ones(1000, F32))
    params = dev(np.full(1000, 3.0, F32))
    for k in range(1, 4):
        call("anode_gpu_online_discount_packed_f32", 1000, 0.5, grad, buf)
        assert np.all(host(buf) == F32(2.0 - 2.0 ** (1 - k)))
    call("anode_gpu_online_add_packed_f32", 1000, -0.25, buf, params)
    assert np.all(host(params) == F32(3.0 - 0.25 * 1.75))
