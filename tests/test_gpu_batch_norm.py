"""GPU parity: the 17 batch-norm entry points through the C ABI against the
oracle, on shapes that reach every tiling of the reducer and every access
width of the maps (aligned and element-aligned pointers, S odd, S == 1, S
larger than a tile, many channels, few channels).
"""
import numpy as np
import pytest
import torch

from gpu_util import F32, assert_bit_exact, assert_close, call, cfg, dev, empty, host, rms

pytestmark = pytest.mark.gpu

# (S, C, N): dim0, dim1, dim2 of the ABI
SHAPES = [
    (784, 16, 32),    # BASELINE config 0
    (49, 20, 6),      # one tile of whole channels, S odd, 16-byte path
    (49, 300, 4),     # several channel tiles, S odd
    (49, 3, 5),       # C*S odd: element path
    (1, 37, 11),      # S == 1
    (1, 1000, 64),
    (1, 512, 40), (2, 6, 33), (3, 8, 17), (1, 4, 16), (2, 64, 100), (3, 4, 15),   # channels shorter than a 16-byte group
    (2, 5, 3),
    (16, 300, 3),     # more channels than a tile may hold
    (7, 513, 2),
    (3000, 2, 2),     # one channel per tile, below the chunk threshold
    (465, 4, 1),      # 16-byte accesses, C*S beyond one pass of a workgroup's lanes, C within the channel unit
    (465, 4, 3),
    (4096, 2, 3),
    (5000, 3, 4),     # chunk tiles, several samples per tile
    (5001, 2, 3),     # chunk tiles, S odd: element path
    (40000, 2, 1),    # a run split over several chunk tiles
    (12544, 4, 8),    # the 112x112 run length of config 2a
]


def make(S, C, N, seed):
    g = np.random.default_rng(seed)
    n = S * C * N
    x = (2 + 3 * g.standard_normal(n)).astype(F32)
    dy = g.standard_normal(n).astype(F32)
    return x, dy


@pytest.mark.parametrize("S,C,N", SHAPES)
@pytest.mark.parametrize("offset", [0, 1])
def test_batch_norm_all_symbols(oracle, S, C, N, offset):
    print(f"case S={S} C={C} N={N} offset={offset}", flush=True)
    eps = 1e-5
    x, dy = make(S, C, N, seed=S * 31 + C)
    n = x.size
    g = np.random.default_rng(7)
    old = g.standard_normal(n).astype(F32)
    oldc = g.standard_normal(C).astype(F32)
    dvar_in = g.standard_normal(C).astype(F32)
    dmean_in = g.standard_normal(C).astype(F32)

    xd, dyd = dev(x, offset), dev(dy, offset)
    dims = (S, C, N)

    # ---- forward ----
    mean_d = empty(C, offset=offset)
    call("anode_gpu_batch_mean_3d1_packed_f32", *dims, xd, mean_d)
    mean = host(mean_d)
    assert_close(mean, oracle.batch_mean(*dims, x, f64=True), "mean")

    var_d = empty(C, offset=offset)
    call("anode_gpu_batch_var_3d1_packed_f32", *dims, eps, xd, mean_d, var_d)
    var = host(var_d)
    assert_close(var, oracle.batch_var(*dims, eps, x, mean, f64=True), "var")

    y_d = empty(n, offset=offset)
    call("anode_gpu_batch_norm_3d1_packed_f32", *dims, xd, mean_d, var_d, y_d)
    y = host(y_d)
    y64 = oracle.batch_norm(*dims, x, mean, var, f64=True)
    assert_close(y, y64, "norm", abs_floor=1e-6 * rms(y64))
    assert_bit_exact(y, oracle.batch_norm(*dims, x, mean, var), "norm vs fp32 restatement")

    # ---- backward reductions, assign then accumulate ----
    for acc in (False, True):
        sfx = "_accumulate" if acc else ""
        seed_c = oldc if acc else None

        out = dev(oldc, offset) if acc else empty(C, offset=offset)
        call(f"anode_gpu_batch_norm_bwd_mean_3d1_packed{sfx}_f32", *dims, dyd, var_d, out)
        ref = oracle.batch_norm_bwd_mean(*dims, dy, var, dmean_in=seed_c, f64=True)
        assert_close(host(out), ref, f"norm_bwd_mean{sfx}", abs_floor=1e-6 * rms(ref))

        out = dev(oldc, offset) if acc else empty(C, offset=offset)
        call(f"anode_gpu_batch_norm_bwd_var_3d1_packed{sfx}_f32", *dims, dyd, xd, mean_d, var_d, out)
        ref = oracle.batch_norm_bwd_var(*dims, dy, x, mean, var, dvar_in=seed_c, f64=True)
        assert_close(host(out), ref, f"norm_bwd_var{sfx}", abs_floor=1e-6 * rms(ref))

        out = dev(oldc, offset) if acc else empty(C, offset=offset)
        call(f"anode_gpu_batch_norm_bwd_var_v2_3d1_packed{sfx}_f32", *dims, dyd, y_d, var_d, out)
        ref = oracle.batch_norm_bwd_var_v2(*dims, dy, y, var, dvar_in=seed_c, f64=True)
        assert_close(host(out), ref, f"norm_bwd_var_v2{sfx}", abs_floor=1e-6 * rms(ref))

        out = dev(oldc, offset) if acc else empty(C, offset=offset)
        call(f"anode_gpu_batch_var_bwd_mean_3d1_packed{sfx}_f32", *dims, dev(dvar_in), xd, mean_d, out)
        ref = oracle.batch_var_bwd_mean(*dims, dvar_in, x, mean, dmean_in=seed_c, f64=True)
        # this sum is ~ n * (rounding error of the fp32 mean), i.e. tiny but not noise: both sides
        # form it in fp64 from the same fp32 inputs, so the relative bar applies (floor for an exact 0)
        assert_close(host(out), ref, f"var_bwd_mean{sfx}", abs_floor=1e-10)

    # ---- backward maps, assign then accumulate ----
    for acc in (False, True):
        sfx = "_accumulate" if acc else ""
        seed = old if acc else None

        out = dev(old, offset) if acc else empty(n, offset=offset)
        call(f"anode_gpu_batch_norm_bwd_3d1_packed{sfx}_f32", *dims, dyd, var_d, out)
        ref = oracle.batch_norm_bwd(*dims, dy, var, dx_in=seed, f64=True)
        assert_close(host(out), ref, f"norm_bwd{sfx}", abs_floor=1e-6 * rms(ref))
        assert_bit_exact(host(out), oracle.batch_norm_bwd(*dims, dy, var, dx_in=seed), f"norm_bwd{sfx} vs fp32")

        out = dev(old, offset) if acc else empty(n, offset=offset)
        call(f"anode_gpu_batch_var_bwd_3d1_packed{sfx}_f32", *dims, dev(dvar_in), xd, mean_d, out)
        ref = oracle.batch_var_bwd(*dims, dvar_in, x, mean, dx_in=seed, f64=True)
        assert_close(host(out), ref, f"var_bwd{sfx}", abs_floor=1e-6 * rms(ref))
        assert_bit_exact(host(out), oracle.batch_var_bwd(*dims, dvar_in, x, mean, dx_in=seed), f"var_bwd{sfx} vs fp32")

        out = dev(old, offset) if acc else empty(n, offset=offset)
        call(f"anode_gpu_batch_mean_bwd_3d1_packed{sfx}_f32", *dims, dev(dmean_in), out)
        ref = oracle.batch_mean_bwd(*dims, dmean_in, dx_in=seed, f64=True)
        assert_close(host(out), ref, f"mean_bwd{sfx}", abs_floor=1e-6 * rms(ref))
        assert_bit_exact(host(out), oracle.batch_mean_bwd(*dims, dmean_in, dx_in=seed), f"mean_bwd{sfx} vs fp32")


def test_batch_norm_recipe_matches_autograd(oracle):
    """The launch sequence anode's graph makes for BN forward + backward
    (src/ops.rs:999-1014; adjoints src/ops_gpu.rs:4344-4352, 3997-4004, 3787-3795):
    first writer assigns, later writers accumulate.  Checked against float64
    torch autograd of batch_norm."""
    N, C, H, W = 8, 6, 14, 14
    S = H * W
    eps = 1e-5
    g = np.random.default_rng(3)
    x = (2 + 3 * g.standard_normal((N, C, H, W))).astype(F32)
    dy = g.standard_normal((N, C, H, W)).astype(F32)
    xd, dyd = dev(x), dev(dy)
    dims = (S, C, N)
    mean, var = empty(C), empty(C)
    y, dx = empty(x.size), empty(x.size)
    dmean, dvar = empty(C), empty(C)
    call("anode_gpu_batch_mean_3d1_packed_f32", *dims, xd, mean)
    call("anode_gpu_batch_var_3d1_packed_f32", *dims, eps, xd, mean, var)
    call("anode_gpu_batch_norm_3d1_packed_f32", *dims, xd, mean, var, y)
    call("anode_gpu_batch_norm_bwd_3d1_packed_f32", *dims, dyd, var, dx)                       # adj_x: assign
    call("anode_gpu_batch_norm_bwd_mean_3d1_packed_f32", *dims, dyd, var, dmean)               # adj_mean: assign
    call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", *dims, dyd, xd, mean, var, dvar)       # adj_var: assign
    call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *dims, dvar, xd, mean, dx)        # adj_x += ...
    call("anode_gpu_batch_var_bwd_mean_3d1_packed_accumulate_f32", *dims, dvar, xd, mean, dmean)
    call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", *dims, dmean, dx)

    xt = torch.from_numpy(x).double().requires_grad_(True)
    yt = torch.nn.functional.batch_norm(xt, None, None, training=True, eps=eps)
    (gx,) = torch.autograd.grad(yt, xt, torch.from_numpy(dy).double())
    assert_close(host(y).reshape(x.shape), yt.detach().numpy(), "y", abs_floor=2e-6)
    gx = gx.numpy()
    assert_close(host(dx).reshape(x.shape), gx, "dx", abs_floor=2e-6 * float(np.abs(gx).max()))


def test_batch_norm_is_reproducible_and_cfg_is_only_a_hint(oracle):
    S, C, N = 3136, 8, 4
    x, _ = make(S, C, N, 5)
    xd = dev(x)
    outs = []
    for block, max_blocks in [(1024, 1024), (32, 7), (1, 1), (2048, 100000)]:
        m = empty(C)
        call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, xd, m, cfg=cfg(block, max_blocks))
        outs.append(host(m).copy())
    for o in outs[1:]:
        assert_bit_exact(o, outs[0], "mean under different KernelConfig")


def test_batch_norm_on_a_side_stream(oracle):
    S, C, N = 784, 16, 8
    x, _ = make(S, C, N, 6)
    xd = dev(x)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    m, v = empty(C), empty(C)
    torch.cuda.synchronize()
    call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, xd, m, stream=side.cuda_stream)
    call("anode_gpu_batch_var_3d1_packed_f32", S, C, N, 1e-5, xd, m, v, stream=side.cuda_stream)
    side.synchronize()
    assert_close(host(m), oracle.batch_mean(S, C, N, x, f64=True), "mean on a side stream")
    assert_close(host(v), oracle.batch_var(S, C, N, 1e-5, x, host(m), f64=True), "var on a side stream")
    # the null stream handle is accepted as well
    m0 = empty(C)
    call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, xd, m0, stream=0)
    assert_bit_exact(host(m0), host(m), "null stream")


@pytest.mark.parametrize("S,C,N", [(784, 16, 8), (49, 40, 16), (3136, 4, 3), (12544, 3, 2), (4, 64, 50), (1, 300, 40)])
def test_batch_norm_arrays_that_lie_differently(oracle, S, C, N):
    # the 16-byte forms need every array of a launch on a 16-byte boundary; with any mix of element offsets the
    # element-wide forms must give the same results, and nothing outside the outputs may be written
    import torch
    eps = 1e-5
    x, dy = make(S, C, N, seed=S + 13 * C)
    n = x.size
    dims = (S, C, N)
    mean = oracle.batch_mean(*dims, x)
    var = oracle.batch_var(*dims, eps, x, mean)
    dvar = np.random.default_rng(3).standard_normal(C).astype(F32)
    old = np.random.default_rng(4).standard_normal(n).astype(F32)

    def guarded(values_or_count, off, fill=4242.0):
        count = values_or_count if isinstance(values_or_count, int) else values_or_count.size
        buf = torch.full((count + 40,), fill, dtype=torch.float32, device="cuda")
        view = buf[16 + off:16 + off + count]
        if not isinstance(values_or_count, int):
            view.copy_(torch.from_numpy(values_or_count))
        return buf, view

    def intact(buf, count, off, fill=4242.0):
        h = host(buf)
        return bool(np.all(h[:16 + off] == fill) and np.all(h[16 + off + count:] == fill))

    for off_x, off_dy, off_out in [(0, 0, 1), (1, 0, 0), (0, 2, 0), (3, 1, 2), (2, 2, 0)]:
        print(f"case S={S} C={C} N={N} offsets {off_x} {off_dy} {off_out}", flush=True)
        xd, dyd = dev(x, off_x), dev(dy, off_dy)
        md, vd = dev(mean, off_dy), dev(var, off_x)
        ybuf, y = guarded(n, off_out)
        call("anode_gpu_batch_norm_3d1_packed_f32", *dims, xd, md, vd, y)
        assert intact(ybuf, n, off_out)
        assert_bit_exact(host(y), oracle.batch_norm(*dims, x, mean, var), "norm")
        abuf, acc = guarded(old, off_out)
        call("anode_gpu_batch_var_bwd_3d1_packed_accumulate_f32", *dims, dev(dvar, off_out), xd, md, acc)
        assert intact(abuf, n, off_out)
        assert_bit_exact(host(acc), oracle.batch_var_bwd(*dims, dvar, x, mean, dx_in=old), "var_bwd accumulate")
        cbuf, out = guarded(C, off_out)
        call("anode_gpu_batch_mean_3d1_packed_f32", *dims, xd, out)
        assert intact(cbuf, C, off_out)
        assert_close(host(out), oracle.batch_mean(*dims, x, f64=True), "mean")
        cbuf, out = guarded(C, off_out)
        call("anode_gpu_batch_norm_bwd_var_3d1_packed_f32", *dims, dyd, xd, md, vd, out)
        assert intact(cbuf, C, off_out)
        ref = oracle.batch_norm_bwd_var(*dims, dy, x, mean, var, f64=True)
        assert_close(host(out), ref, "norm_bwd_var", abs_floor=1e-6 * rms(ref))
