"""The entry points under HIP graph capture: a batch-norm layer (forward + backward, nine launches plus the
reductions' fold kernels) and a softmax + NLL head are captured once and replayed on changing inputs, with eager work
and synchronisations between the replays; every replay must equal the eager result to the bit.

The reductions keep their partial-sum buffer per (device, stream) and allocate it on first use, so the sequence is
run once on the capture stream before capture (allocation is not possible while capturing).
"""
import ctypes

import numpy as np
import pytest
import torch

from gpu_util import F32, assert_bit_exact, call, dev, empty, host

pytestmark = pytest.mark.gpu


def _bn_layer(d, x, dy, bufs):
    mean, var, y, dx, dmean, dvar = bufs
    call("anode_gpu_batch_mean_3d1_packed_f32", *d, x, mean)
    call("anode_gpu_batch_var_3d1_packed_f32", *d, 1e-5, x, mean, var)
    call("anode_gpu_batch_norm_3d1_packed_f32", *d, x, mean, var, y)
    call("anode_gpu_positive_clip_flat_map_f32", d[0] * d[1] * d[2], y, y)
    call("anode_gpu_batch_norm_bwd_3d1_packed_f32", *d, dy, var, dx)
    call("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", *d, dy, var, dmean)
    call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", *d, dy, x, mean, var, dvar)
    call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *d, dvar, x, mean, dx)
    call("anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", *d, dvar, x, mean, dmean)
    call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", *d, dmean, dx)


def _head(K, R, logits, labels, ones, bufs):
    p, nll, dl = bufs
    call("anode_gpu_softmax_packed_block_f32", K, R, logits, p)
    call("anode_gpu_softmax_cat_nll_packed_f32", K, R, p, labels, nll)
    call("anode_gpu_softmax_cat_nll_bwd_packed_f32", K, R, ones, p, labels, dl)


@pytest.mark.parametrize("d", [(784, 16, 32), (49, 256, 64)])
def test_graph_replay_equals_eager(d):
    S, C, N = d
    n = S * C * N
    K, R = 1000, 64
    g = np.random.default_rng(S)
    stream = torch.cuda.Stream()
    x, dy = empty(n), empty(n)
    logits, labels, ones = empty(K * R), dev(g.integers(0, K, R).astype(np.uint32)), dev(np.ones(R, F32))

    def buffers():
        return ([empty(C), empty(C), empty(n), empty(n), empty(C), empty(C)], [empty(K * R), empty(R), empty(K * R)])

    def refill(seed):
        r = np.random.default_rng(seed)
        x.copy_(torch.from_numpy((2 + 3 * r.standard_normal(n)).astype(F32)))
        dy.copy_(torch.from_numpy(r.standard_normal(n).astype(F32)))
        logits.copy_(torch.from_numpy((2 * r.standard_normal(K * R)).astype(F32)))
        torch.cuda.synchronize()

    gb, gh = buffers()
    refill(0)
    with torch.cuda.stream(stream):          # warm-up on the capture stream: allocates the reduction scratch
        _bn_layer(d, x, dy, gb)
        _head(K, R, logits, labels, ones, gh)
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        _bn_layer(d, x, dy, gb)
        _head(K, R, logits, labels, ones, gh)

    for seed in (1, 2, 3, 4):
        refill(seed)
        eb, eh = buffers()
        _bn_layer(d, x, dy, eb)              # eager, on the default stream, into separate outputs
        _head(K, R, logits, labels, ones, eh)
        torch.cuda.synchronize()
        for t in gb + gh:
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(gb + gh, eb + eh):
            assert_bit_exact(host(got), host(want), f"replay with seed {seed}")


def test_capture_without_scratch_is_refused_and_reserve_makes_it_work():
    # A reduction whose channels are cut into several tiles needs the stream's partial-sum buffer.  Allocating it is
    # impossible while the stream is being captured: the call must enqueue nothing, record
    # hipErrorStreamCaptureUnsupported (900) and leave the capture valid.  After anode_gpu_reserve_scratch the same
    # capture works and its replays equal the eager result.
    from anode_amd import gpu
    from anode_amd._lib import load

    lib = load()
    d = (12544, 8, 16)
    S, C, N = d
    g = np.random.default_rng(5)
    x = dev((2 + 3 * g.standard_normal(S * C * N)).astype(F32))
    mean, marker, want = empty(C), empty(4), empty(C)
    stream = torch.cuda.Stream()
    handle = ctypes.c_void_p(stream.cuda_stream)
    stream.synchronize()
    lib.symbol("anode_gpu_release_scratch")(handle)      # torch hands out pooled streams: drop what an earlier test left

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        marker.fill_(1.0)
        gpu.call("anode_gpu_batch_mean_3d1_packed_f32", *d, x, mean)
        err = gpu.take_last_error()
    assert err == 900, err
    graph.replay()
    torch.cuda.synchronize()
    assert np.all(host(marker) == 1.0) and np.all(np.isnan(host(mean)))   # the capture survived; nothing was enqueued

    need = lib.symbol("anode_gpu_reduce_scratch_bytes")(*d)
    assert need > 0
    assert lib.symbol("anode_gpu_reserve_scratch")(handle, need) == 0
    graph2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph2, stream=stream):
        call("anode_gpu_batch_mean_3d1_packed_f32", *d, x, mean)
    call("anode_gpu_batch_mean_3d1_packed_f32", *d, x, want)
    for k in range(3):
        mean.fill_(float("nan"))
        torch.cuda.synchronize()
        graph2.replay()
        torch.cuda.synchronize()
        assert_bit_exact(host(mean), host(want), f"replay {k}")
    stream.synchronize()
    assert lib.symbol("anode_gpu_release_scratch")(handle) >= 1
