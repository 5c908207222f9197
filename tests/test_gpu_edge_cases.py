"""Empty and degenerate shapes through every entry point the header declares: all dimensions zero, and each
dimension zero in turn.  Nothing may fault, no launch error may be recorded, and nothing may be written outside the
(empty or tiny) arrays.  With every dimension zero the call must leave all buffers untouched -- except the scalar sum,
whose result for an empty array is 0 by definition.
"""
import ctypes

import numpy as np
import pytest
import torch

from anode_amd import gpu
from anode_amd._lib import load
from gpu_util import F32, assert_bit_exact, assert_close, call, dev, host

pytestmark = pytest.mark.gpu

SENTINEL = 12345.0
WRITES_ON_EMPTY = {"anode_gpu_sum_packed_deterministic_f32", "gpudevicemem_sum_packed_deterministic_f32"}


def _entry_points():
    lib = load()  # operators only: everything that ends in (cfg, stream)
    return sorted(n for n, (_, _, names) in lib.prototypes.items()
                  if n.startswith(("anode_gpu_", "gpudevicemem_")) and names[-2:] == ["cfg", "stream"])


def _call(name, dims):
    lib = load()
    _, argtypes, names = lib.prototypes[name]
    dims = iter(dims)
    bufs, args = [], []
    for t, _ in zip(argtypes[:-2], names[:-2]):
        if t is ctypes.c_uint32:
            args.append(next(dims))
        elif t is ctypes.c_float:
            args.append(0.5)
        else:
            b = torch.full((64,), SENTINEL, device="cuda")
            bufs.append(b)
            args.append(b)
    gpu.call(name, *args)
    torch.cuda.synchronize()
    return bufs


def _n_dims(name):
    return sum(1 for t in load().prototypes[name][1][:-2] if t is ctypes.c_uint32)


@pytest.mark.parametrize("name", _entry_points())
def test_all_dimensions_zero_is_a_no_op(name):
    bufs = _call(name, [0] * _n_dims(name))
    assert gpu.take_last_error() == 0
    if name in WRITES_ON_EMPTY:
        return
    for b in bufs:
        assert bool((b == SENTINEL).all()), f"{name} wrote to a buffer although every dimension is zero"


@pytest.mark.parametrize("name", _entry_points())
def test_each_dimension_zero_in_turn(name):
    nd = _n_dims(name)
    for zero_at in range(nd):
        dims = [3] * nd
        dims[zero_at] = 0
        bufs = _call(name, dims)
        assert gpu.take_last_error() == 0, (name, dims)
        for b in bufs:  # at most 3*3*3 elements belong to the arrays
            assert bool((b[32:] == SENTINEL).all()), f"{name}{dims} wrote past the end of an array"


# A reduction over no elements still writes every channel: the reference runs one block per channel whatever the
# extent of the reduced axes (routines_gpu/batch_norm.cu:35-56: zero tiles, then mean[c] = 0 / 0).
@pytest.mark.parametrize("S,C,N", [(0, 5, 3), (7, 5, 0), (0, 300, 0)])
def test_reductions_over_an_empty_axis_write_every_channel(oracle, S, C, N):
    g = np.random.default_rng(C)
    x = np.zeros(0, F32)
    mean = g.standard_normal(C).astype(F32)
    var = (0.5 + g.random(C)).astype(F32)
    dvar = g.standard_normal(C).astype(F32)
    old = g.standard_normal(C).astype(F32)
    xd = torch.empty(16, device="cuda")
    d = (S, C, N)

    def run(name, *args):
        out = dev(old)
        call(name, *d, *args, out)
        return host(out)

    assert_close(run("anode_gpu_batch_mean_3d1_packed_f32", xd), oracle.batch_mean(*d, x), "mean")
    assert np.all(np.isnan(run("anode_gpu_batch_mean_3d1_packed_f32", xd)))
    assert_close(run("anode_gpu_batch_var_3d1_packed_f32", 1e-5, xd, dev(mean)),
                     oracle.batch_var(*d, 1e-5, x, mean), "var")
    assert_close(run("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", xd, dev(var)),
                     oracle.batch_norm_bwd_mean(*d, x, var), "norm_bwd_mean")
    assert_close(run("anode_gpu_batch_norm_bwd_mean_3d1_packed_accumulate_f32", xd, dev(var)),
                     oracle.batch_norm_bwd_mean(*d, x, var, dmean_in=old), "norm_bwd_mean accumulate")
    assert_close(run("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", xd, xd, dev(mean), dev(var)),
                     oracle.batch_norm_bwd_var(*d, x, x, mean, var), "norm_bwd_var")
    assert_close(run("anode_gpu_batch_norm_bwd_var_3d1_packed_accumulate_f32", xd, xd, dev(mean), dev(var)),
                     oracle.batch_norm_bwd_var(*d, x, x, mean, var, dvar_in=old), "norm_bwd_var accumulate")
    assert_close(run("anode_gpu_batch_norm_bwd_var_v2_3d1_packed_f32", xd, xd, dev(var)),
                     oracle.batch_norm_bwd_var_v2(*d, x, x, var), "norm_bwd_var_v2")
    assert_close(run("anode_gpu_batch_var_bwd_mean_3d1_packed_f32", dev(dvar), xd, dev(mean)),
                     oracle.batch_var_bwd_mean(*d, dvar, x, mean), "var_bwd_mean")
    assert_close(run("anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", dev(dvar), xd, dev(mean)),
                     oracle.batch_var_bwd_mean(*d, dvar, x, mean, dmean_in=old), "var_bwd_mean accumulate")


def test_f1_over_no_positions_is_minus_one(oracle):
    K, N = 4, 3
    y = dev(np.full(K * N, 7.0, F32))
    xd = torch.empty(16, device="cuda")
    call("anode_gpu_smooth_negative_f1_loss_3d1_packed_f32", 0, K, N, 0.25, xd, xd, y)
    got = host(y)
    assert_bit_exact(got, oracle.f1_loss(0, K, N, 0.25, np.zeros(0, F32), np.zeros(0, F32)), "f1 over nothing")
    assert np.all(got == -1.0)  # -(2*0 + eps) / (0 + eps)
