"""The entry point that allocates nothing: anode_gpu_batch_mean_var_3d1_packed_noalloc_f32 keeps its partial sums
in a device array that is part of the library image.  Its output must equal that of the allocating entry point,
anode_gpu_batch_mean_var_3d1_packed_f32, to the bit (same kernels, same tiling), also on a second call with a
smaller input, which finds the first call's partial sums still in the array."""
import ctypes

import numpy as np
import pytest
import torch

from anode_amd import gpu
from anode_amd._lib import load
from gpu_util import F32, assert_bit_exact, assert_close, call, dev, empty, host

pytestmark = pytest.mark.gpu

NOALLOC = "anode_gpu_batch_mean_var_3d1_packed_noalloc_f32"
PLAIN = "anode_gpu_batch_mean_var_3d1_packed_f32"


def _noalloc(S, C, N, eps, x, mean, var, stream=None):
    lib = load()
    if stream is None:
        stream = torch.cuda.current_stream().cuda_stream
    rc = lib.symbol(NOALLOC)(S, C, N, eps, x.data_ptr(), mean.data_ptr(), var.data_ptr(),
                             ctypes.byref(gpu.DEFAULT_CONFIG), ctypes.c_void_p(stream))
    assert gpu.take_last_error() == 0
    return rc


def _one(oracle, S, C, N, seed, offset=0):
    print(f"noalloc case S={S} C={C} N={N} seed={seed} offset={offset}", flush=True)
    g = np.random.default_rng(seed)
    x = (2 + 3 * g.standard_normal(S * C * N)).astype(F32)
    xd = dev(x, offset)
    mean_a, var_a, mean_b, var_b = empty(C), empty(C), empty(C), empty(C)
    assert _noalloc(S, C, N, 1e-5, xd, mean_a, var_a) == 0
    call(PLAIN, S, C, N, 1e-5, xd, mean_b, var_b)
    assert_bit_exact(host(mean_a), host(mean_b), f"mean [{S},{C},{N}]")
    assert_bit_exact(host(var_a), host(var_b), f"var [{S},{C},{N}]")
    m64, v64 = oracle.batch_mean_var(S, C, N, 1e-5, x)
    assert_close(host(mean_a), m64, "mean vs fp64 oracle")
    assert_close(host(var_a), v64, "var vs fp64 oracle")


def test_captured_into_a_graph_on_a_stream_without_scratch():
    # The callers this entry point is for: a stream under HIP graph capture that holds no reduction scratch.  There
    # the allocating entry point is refused (error 900, nothing enqueued) while this one is captured -- in a fresh
    # process this is also its first call on the device, so the address of the static array is looked up during the
    # capture -- and every replay equals the eager result to the bit.  [12544, 8, 16] cuts its channels into several
    # tiles, so the partial sums do go through the array.
    lib = load()
    d = (12544, 8, 16)
    S, C, N = d
    assert lib.symbol("anode_gpu_reduce_scratch_bytes")(*d) > 0
    g = np.random.default_rng(11)
    x = dev((2 + 3 * g.standard_normal(S * C * N)).astype(F32))
    mean, var, refused = empty(C), empty(C), empty(C)
    stream = torch.cuda.Stream()
    handle = ctypes.c_void_p(stream.cuda_stream)
    stream.synchronize()
    lib.symbol("anode_gpu_release_scratch")(handle)      # torch hands out pooled streams: drop what an earlier test left
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        gpu.call("anode_gpu_batch_mean_3d1_packed_f32", *d, x, refused)
        err_plain = gpu.take_last_error()
        rc = lib.symbol(NOALLOC)(S, C, N, 1e-5, x.data_ptr(), mean.data_ptr(), var.data_ptr(),
                                 ctypes.byref(gpu.DEFAULT_CONFIG), handle)
        err = gpu.take_last_error()
    assert err_plain == 900, err_plain
    assert rc == 0 and err == 0, (rc, err)
    want_mean, want_var = empty(C), empty(C)
    call(PLAIN, S, C, N, 1e-5, x, want_mean, want_var)   # eager, default stream
    for k in range(3):
        mean.fill_(float("nan"))
        var.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert_bit_exact(host(mean), host(want_mean), f"mean, replay {k}")
        assert_bit_exact(host(var), host(want_var), f"var, replay {k}")
        x.mul_(1.5)                                      # eager work between the replays, on changing input
        call(PLAIN, S, C, N, 1e-5, x, want_mean, want_var)
    assert np.all(np.isnan(host(refused)))
    assert lib.symbol("anode_gpu_release_scratch")(handle) == 0   # the stream never got a buffer


def test_two_calls_in_a_row_second_smaller(oracle):
    # first call: many tiles per channel (chunk tiles); second: fewer and smaller partial lists in the same array,
    # which still holds the first call's sums
    _one(oracle, 12544, 16, 32, seed=1)
    _one(oracle, 49, 40, 24, seed=2)
    _one(oracle, 5000, 3, 5, seed=3, offset=1)   # element-aligned input
    _one(oracle, 7, 5, 1, seed=4)                # one tile per channel: no partial sums at all


def test_stream_order_keeps_calls_apart():
    # back-to-back calls on one stream share the array; stream order is enough
    S, C, N = 784, 16, 64
    g = np.random.default_rng(7)
    xs = [dev((k + g.standard_normal(S * C * N)).astype(F32)) for k in range(4)]
    outs = [(empty(C), empty(C)) for _ in xs]
    refs = [(empty(C), empty(C)) for _ in xs]
    for x, (m, v) in zip(xs, outs):
        assert _noalloc(S, C, N, 1e-5, x, m, v) == 0
    for x, (m, v) in zip(xs, refs):
        call(PLAIN, S, C, N, 1e-5, x, m, v)
    for (m, v), (rm, rv) in zip(outs, refs):
        assert_bit_exact(host(m), host(rm), "mean")
        assert_bit_exact(host(v), host(rv), "var")


def test_calls_on_two_streams_are_put_in_order():
    # Calls on different streams of one GPU share the array; outside graph capture the library orders them on the
    # device (each call waits for the event the previous call recorded behind its kernels), so neither stream's
    # partial sums are overwritten while its second kernel still reads them.  Two streams, no host synchronisation
    # in between, a long and a short reduction in turn, thirty rounds; every result against the allocating entry point.
    big, small = (12544, 16, 32), (784, 16, 64)
    g = np.random.default_rng(21)
    xa = dev((1 + g.standard_normal(big[0] * big[1] * big[2])).astype(F32))
    xb = dev((2 + g.standard_normal(small[0] * small[1] * small[2])).astype(F32))
    sa, sb = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    rounds = 30
    outs_a = [(empty(big[1]), empty(big[1])) for _ in range(rounds)]
    outs_b = [(empty(small[1]), empty(small[1])) for _ in range(rounds)]
    torch.cuda.synchronize()
    for k in range(rounds):
        assert _noalloc(*big, 1e-5, xa, *outs_a[k], stream=sa.cuda_stream) == 0
        assert _noalloc(*small, 1e-5, xb, *outs_b[k], stream=sb.cuda_stream) == 0
    sa.synchronize()
    sb.synchronize()
    ref_a, ref_b = (empty(big[1]), empty(big[1])), (empty(small[1]), empty(small[1]))
    call(PLAIN, *big, 1e-5, xa, *ref_a)
    call(PLAIN, *small, 1e-5, xb, *ref_b)
    for k in range(rounds):
        assert_bit_exact(host(outs_a[k][0]), host(ref_a[0]), f"mean, long reduction, round {k}")
        assert_bit_exact(host(outs_a[k][1]), host(ref_a[1]), f"var, long reduction, round {k}")
        assert_bit_exact(host(outs_b[k][0]), host(ref_b[0]), f"mean, short reduction, round {k}")
        assert_bit_exact(host(outs_b[k][1]), host(ref_b[1]), f"var, short reduction, round {k}")


def test_oversized_shape_is_refused():
    # With lane tiles switched off (tuning knob 9), [1, 65536, 4096] is cut into 32 sample tiles: 32 partials for
    # each of 65536 channels, two sums -> 32 MiB > 4 MiB.  The call must return 1 and enqueue nothing.  The buffers
    # have their full size all the same: a call that were accepted would only compute, never touch foreign memory.
    S, C, N = 1, 65536, 4096
    x = torch.empty(S * C * N, device="cuda")
    mean, var = empty(C), empty(C)
    saved = gpu.set_tuning(9, 0)
    try:
        assert load().symbol("anode_gpu_reduce_scratch_bytes")(S, C, N) > (4 << 20)
        rc = _noalloc(S, C, N, 1e-5, x, mean, var)
    finally:
        gpu.set_tuning(9, saved)
    torch.cuda.synchronize()
    assert rc == 1
    assert np.all(np.isnan(host(mean))) and np.all(np.isnan(host(var)))
