"""Empty and degenerate shapes through every entry point the header declares: all dimensions zero, and each
dimension zero in turn.  Nothing may fault, no launch error may be recorded, and nothing may be written outside the
(empty or tiny) arrays.  With every dimension zero the call must leave all buffers untouched -- except the scalar sum,
whose result for an empty array is 0 by definition.
"""
import ctypes
import itertools

import pytest
import torch

from anode_amd import gpu
from anode_amd._lib import load

pytestmark = pytest.mark.gpu

SENTINEL = 12345.0
WRITES_ON_EMPTY = {"anode_gpu_sum_packed_deterministic_f32"}


def _entry_points():
    lib = load()
    return sorted(n for n in lib.prototypes if n.startswith("anode_gpu_") and n not in
                  ("anode_gpu_take_last_error", "anode_gpu_reference_symbol_count"))


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
