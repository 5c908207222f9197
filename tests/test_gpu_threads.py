"""Re-entrancy: anode calls the library from several host threads, each with its own stream
(src/context.rs:40-62: the context is thread-local).  The reductions' scratch cache is shared state inside the
library; concurrent callers on different streams must get the results a single caller gets, to the bit.
"""
import threading

import numpy as np
import pytest
import torch

from gpu_util import F32, assert_bit_exact, call, dev, empty, host

pytestmark = pytest.mark.gpu

SHAPES = [(49, 64, 32), (3136, 16, 8), (1, 24, 500), (20000, 3, 5)]


def _layer(d, x, dy):
    S, C, N = d
    n = S * C * N
    mean, var, y, dx, dmean, dvar = empty(C), empty(C), empty(n), empty(n), empty(C), empty(C)
    call("anode_gpu_batch_mean_3d1_packed_f32", *d, x, mean)
    call("anode_gpu_batch_var_3d1_packed_f32", *d, 1e-5, x, mean, var)
    call("anode_gpu_batch_norm_3d1_packed_f32", *d, x, mean, var, y)
    call("anode_gpu_batch_norm_bwd_3d1_packed_f32", *d, dy, var, dx)
    call("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", *d, dy, var, dmean)
    call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", *d, dy, x, mean, var, dvar)
    call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *d, dvar, x, mean, dx)
    call("anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", *d, dvar, x, mean, dmean)
    call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", *d, dmean, dx)
    return mean, var, y, dx, dmean, dvar


def test_concurrent_callers_on_their_own_streams():
    g = np.random.default_rng(5)
    inputs = []
    for d in SHAPES:
        n = d[0] * d[1] * d[2]
        inputs.append((d, dev((2 + 3 * g.standard_normal(n)).astype(F32)), dev(g.standard_normal(n).astype(F32))))
    want = [[host(t).copy() for t in _layer(d, x, dy)] for d, x, dy in inputs]
    torch.cuda.synchronize()

    errors = []
    barrier = threading.Barrier(len(inputs))

    def worker(i):
        try:
            d, x, dy = inputs[i]
            stream = torch.cuda.Stream()
            barrier.wait()
            for rep in range(20):
                with torch.cuda.stream(stream):
                    outs = _layer(d, x, dy)
                stream.synchronize()
                for got, ref in zip(outs, want[i]):
                    assert_bit_exact(got.cpu().numpy(), ref, f"thread {i} repetition {rep}")
        except BaseException as e:  # noqa: BLE001 - reported in the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(inputs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_eight_threads_run_config0_layers_on_their_own_streams():
    # BASELINE config 0's batch-norm layer ([32,16,28,28], one launch per reduction) and a layer whose channels are
    # cut into 16 tiles ([16,8,112,112]: partial sums in the stream's buffer, then the fold kernel) from eight host
    # threads at once, each on a stream of its own and with data of its own.  Each stream's buffer has its own lock,
    # so the threads do not wait for each other; every result equals the single-threaded one to the bit.
    shapes = [(784, 16, 32), (12544, 8, 16)]
    g = np.random.default_rng(6)
    inputs = []
    for i in range(8):
        per_thread = []
        for d in shapes:
            n = d[0] * d[1] * d[2]
            per_thread.append((d, dev((i + g.standard_normal(n)).astype(F32)), dev(g.standard_normal(n).astype(F32))))
        inputs.append(per_thread)
    want = [[[host(t).copy() for t in _layer(d, x, dy)] for d, x, dy in per_thread] for per_thread in inputs]
    torch.cuda.synchronize()
    errors = []
    barrier = threading.Barrier(len(inputs))

    def worker(i):
        try:
            stream = torch.cuda.Stream()
            barrier.wait()
            for rep in range(15):
                for k, (d, x, dy) in enumerate(inputs[i]):
                    with torch.cuda.stream(stream):
                        outs = _layer(d, x, dy)
                    stream.synchronize()
                    for got, ref in zip(outs, want[i][k]):
                        assert_bit_exact(got.cpu().numpy(), ref, f"thread {i} shape {d} repetition {rep}")
        except BaseException as e:  # noqa: BLE001 - reported in the main thread
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(len(inputs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_two_threads_share_one_stream():
    # Two host threads enqueue on the same stream: a reduction's two kernels (partial sums, then the fold) must not
    # be interleaved with the other thread's, or one fold would read the other call's partial sums.
    d = (12544, 8, 16)     # 16 tiles per channel: every reduction is two launches
    n = d[0] * d[1] * d[2]
    g = np.random.default_rng(7)
    inputs = [(dev((1 + i + 2 * g.standard_normal(n)).astype(F32)), dev(g.standard_normal(n).astype(F32))) for i in range(2)]
    want = [[host(t).copy() for t in _layer(d, x, dy)] for x, dy in inputs]
    torch.cuda.synchronize()
    stream = torch.cuda.Stream()
    errors = []
    barrier = threading.Barrier(2)

    def worker(i):
        try:
            x, dy = inputs[i]
            barrier.wait()
            for rep in range(25):
                with torch.cuda.stream(stream):
                    outs = _layer(d, x, dy)
                stream.synchronize()
                for got, ref in zip(outs, want[i]):
                    assert_bit_exact(got.cpu().numpy(), ref, f"thread {i} repetition {rep}")
        except BaseException as e:  # noqa: BLE001
            errors.append((i, repr(e)))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(2)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
