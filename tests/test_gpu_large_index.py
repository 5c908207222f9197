"""Arrays of more than 2^31 elements (the ABI's counts are 32-bit, so up to 2^32 - 1): every index computation in the
kernels has to survive element offsets, and offset + grid stride, beyond 2^31 and close to 2^32.

torch is the checker here (same formula on the device; a host copy of 8 GiB arrays would only add minutes): exact
equality for the maps, 1e-5 against float64 for the reductions and the softmax.
"""
import numpy as np
import pytest
import torch

from gpu_util import call

pytestmark = pytest.mark.gpu

N_BIG = (1 << 31) + (1 << 20) + 7   # odd, above 2^31


@pytest.fixture(scope="module")
def big():
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    x = torch.empty(N_BIG + 4, device="cuda")
    x.normal_(generator=g)
    yield x
    del x
    torch.cuda.empty_cache()


@pytest.mark.parametrize("offset", [0, 1])
def test_flat_map_beyond_2_31(big, offset):
    x = big[offset:offset + N_BIG]
    y = torch.full((N_BIG + 4,), float("nan"), device="cuda")
    call("anode_gpu_positive_clip_flat_map_f32", N_BIG, x, y[offset:offset + N_BIG])
    torch.cuda.synchronize()
    assert torch.equal(y[offset:offset + N_BIG], torch.relu(x))
    assert bool(torch.isnan(y[offset + N_BIG:]).all()) and bool(torch.isnan(y[:offset]).all())
    del y


@pytest.mark.parametrize("offset", [0, 1])
def test_accumulate_map_applies_once_beyond_2_31(big, offset):
    x = big[offset:offset + N_BIG]
    y = torch.ones(N_BIG + 4, device="cuda")
    call("anode_gpu_add_packed_f32", N_BIG, x, y[offset:offset + N_BIG])
    torch.cuda.synchronize()
    assert torch.equal(y[offset:offset + N_BIG], x + 1.0)
    assert bool((y[offset + N_BIG:] == 1).all())
    del y


@pytest.mark.parametrize("offset", [0, 1])
def test_batch_norm_pieces_beyond_2_31(big, offset):
    S, C, N = 1 << 20, 3, 683           # 2 148 532 224 elements
    n = S * C * N
    assert (1 << 31) < n <= N_BIG
    x = big[offset:offset + n]
    mean, var = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, x, mean)
    call("anode_gpu_batch_var_3d1_packed_f32", S, C, N, 1e-5, x, mean, var)
    torch.cuda.synchronize()
    xv = x.view(N, C, S)
    for c in range(C):
        col = xv[:, c, :].double()
        m = col.mean().item()
        v = ((col - float(mean[c])) ** 2).mean().item() + 1e-5
        assert abs(float(mean[c]) - m) <= 1e-5 * abs(m) + 1e-7
        assert abs(float(var[c]) - v) <= 1e-5 * v
        del col
    dx = torch.zeros(n + 4, device="cuda")[offset:offset + n]
    dmean = torch.tensor([1.0, 2.0, 3.0], device="cuda") * float(S * N)
    call("anode_gpu_batch_mean_bwd_3d1_packed_accumulate_f32", S, C, N, dmean, dx)
    torch.cuda.synchronize()
    want = torch.tensor([1.0, 2.0, 3.0], device="cuda").view(1, C, 1).expand(N, C, S)
    assert torch.equal(dx.view(N, C, S), want)
    del dx


def test_softmax_nd_beyond_2_31(big):
    P, C, N = 1 << 16, 19, 1725         # 2 147 942 400 elements
    n = P * C * N
    assert (1 << 31) < n <= N_BIG
    x = big[:n]
    p = torch.empty(n, device="cuda")
    call("anode_gpu_softmax_nd_packed_f32", P, C, N, x, p)
    lab = torch.randint(0, C, (P * N,), device="cuda", dtype=torch.int32)
    nll = torch.empty(P * N, device="cuda")
    call("anode_gpu_softmax_nd_cat_nll_packed_f32", P, C, N, p, lab, nll)
    torch.cuda.synchronize()
    pv = p.view(N, C, P)
    for i in (0, N // 2, N - 1):        # float64 checks on single samples (the first, one across 2^31, the last)
        ref = torch.softmax(x.view(N, C, P)[i].double(), dim=0)
        assert bool(((pv[i].double() - ref).abs() <= 1e-5 * ref).all())
        picked = torch.gather(pv[i], 0, lab.view(N, P)[i].long().unsqueeze(0)).squeeze(0)
        assert torch.allclose(nll.view(N, P)[i], -torch.log(picked), rtol=1e-5, atol=1e-6)
    sums = pv.sum(dim=1)
    assert bool(((sums - 1).abs() < 1e-5).all())
    del p, sums


def test_softmax_nd_samples_of_more_than_4_gib(big):
    # Planes of 64 Mi pixels: a sample of 17 planes is 4.5 GB, so the byte offsets of a wave that crosses from one
    # sample into the next (and of the odd lane's plane pitch) no longer fit 32 bits and the two-lane kernel takes
    # its form with 64-bit lane offsets.  Two samples, the plain and the fused forward + backward entry points.
    P, C, N = 1 << 26, 17, 1
    n = P * C * N
    assert n <= N_BIG
    x = big[:n]
    p = torch.empty(n, device="cuda")
    call("anode_gpu_softmax_nd_packed_f32", P, C, N, x, p)
    torch.cuda.synchronize()
    xv, pv = x.view(C, P), p.view(C, P)
    for lo in (0, P // 2 - 4096, P - 8192):                # float64 checks on slices of the pixels
        ref = torch.softmax(xv[:, lo:lo + 8192].double(), dim=0)
        assert bool(((pv[:, lo:lo + 8192].double() - ref).abs() <= 1e-5 * ref).all())
    assert bool(((pv.sum(dim=0) - 1).abs() < 1e-5).all())
    lab = torch.randint(0, C, (P * N,), device="cuda", dtype=torch.int32)
    dy = torch.randn(P * N, device="cuda")
    p2, nll, dx = torch.empty(n, device="cuda"), torch.empty(P * N, device="cuda"), torch.empty(n, device="cuda")
    call("anode_gpu_softmax_nd_cat_nll_fused_fwd_bwd_packed_f32", P, C, N, x, lab, dy, p2, nll, dx)
    torch.cuda.synchronize()
    assert torch.equal(p2, p)
    picked = torch.gather(pv, 0, lab.long().unsqueeze(0)).squeeze(0)
    assert torch.allclose(nll, -torch.log(picked), rtol=1e-5, atol=1e-6)
    ks = torch.arange(C, device="cuda", dtype=torch.int32).view(C, 1)
    for lo in (0, P - 8192):
        sl = slice(lo, lo + 8192)
        want = dy[sl].unsqueeze(0) * (pv[:, sl] - (lab[sl].unsqueeze(0) == ks).float())
        assert torch.equal(dx.view(C, P)[:, sl], want)
    del p, p2, nll, dx, picked


def test_softmax_nd_backward_beyond_2_31(big):
    # planes of up to 131072 pixels: the backward pass walks the array flat, one 16-byte group of dx per thread
    P, C, N = 1 << 16, 19, 1725
    n = P * C * N
    p = big[:n]                          # any values will do as "probabilities": the map is dy * (p - onehot)
    lab = torch.randint(0, C + 1, (P * N,), device="cuda", dtype=torch.int32)   # C itself: out of range
    dy = torch.randn(P * N, device="cuda")
    dx = torch.empty(n, device="cuda")
    call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dy, p, lab, dx)
    torch.cuda.synchronize()
    pv, dv = p.view(N, C, P), dx.view(N, C, P)
    ks = torch.arange(C, device="cuda", dtype=torch.int32).view(C, 1)
    for i in (0, N // 2, N - 1):
        want = dy.view(N, P)[i].unsqueeze(0) * (pv[i] - (lab.view(N, P)[i].unsqueeze(0) == ks).float())
        assert torch.equal(dv[i], want), i
    del dx


def test_softmax_nd_planes_that_are_not_whole_groups_beyond_2_31(big):
    # planes of 65537 pixels: the 16-byte kernels over groups of four pixels whose last one ends with the plane (two
    # lanes per group at 19 classes, column tiles in registers at 220), and the backward pass walked flat in dx's
    # 16-byte groups wherever the planes end
    for P, C, N in ((65537, 19, 1725), (65537, 220, 149)):
        n = P * C * N
        assert (1 << 31) < n <= N_BIG
        x = big[:n]
        p = torch.empty(n + 8, device="cuda")
        p[n:] = 777.0
        call("anode_gpu_softmax_nd_packed_f32", P, C, N, x, p[:n])
        torch.cuda.synchronize()
        assert bool((p[n:] == 777.0).all())
        pv = p[:n].view(N, C, P)
        for i in (0, N // 2, N - 1):
            ref = torch.softmax(x.view(N, C, P)[i].double(), dim=0)
            assert bool(((pv[i].double() - ref).abs() <= 1e-5 * ref).all()), (P, C, i)
        sums = pv.sum(dim=1)
        assert bool(((sums - 1).abs() < 1e-5).all())
        del sums
        lab = torch.randint(0, C + 1, (P * N,), device="cuda", dtype=torch.int32)
        dy = torch.randn(P * N, device="cuda")
        dx = torch.empty(n + 8, device="cuda")
        dx[n:] = 555.0
        call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dy, p[:n], lab, dx[:n])
        torch.cuda.synchronize()
        assert bool((dx[n:] == 555.0).all())
        dv = dx[:n].view(N, C, P)
        ks = torch.arange(C, device="cuda", dtype=torch.int32).view(C, 1)
        for i in (0, N // 2, N - 1):
            want = dy.view(N, P)[i].unsqueeze(0) * (pv[i] - (lab.view(N, P)[i].unsqueeze(0) == ks).float())
            assert torch.equal(dv[i], want), (P, C, i)
        del p, dx, lab, dy


def test_softmax_nd_many_classes_beyond_2_31(big):
    # 220 classes: column tiles in registers (a workgroup per run of 32 pixel groups with all their classes)
    P, C, N = 1 << 16, 220, 149          # 2 148 270 080 elements
    n = P * C * N
    assert (1 << 31) < n <= N_BIG
    x = big[:n]
    p = torch.empty(n, device="cuda")
    call("anode_gpu_softmax_nd_packed_f32", P, C, N, x, p)
    torch.cuda.synchronize()
    pv = p.view(N, C, P)
    for i in (0, N // 2, N - 1):
        ref = torch.softmax(x.view(N, C, P)[i].double(), dim=0)
        assert bool(((pv[i].double() - ref).abs() <= 1e-5 * ref).all())
    sums = pv.sum(dim=1)
    assert bool(((sums - 1).abs() < 1e-5).all())
    del p, sums


def test_short_channels_beyond_2_31(big):
    # 7x7 maps: the reductions run as lane tiles (one launch, all samples per workgroup), the maps walk channels of
    # 49 elements; sample offsets n * C * S pass 2^31
    S, C, N = 49, 2048, 21409            # 2 148 435 968 elements
    n = S * C * N
    assert (1 << 31) < n <= N_BIG
    x = big[:n]
    mean, var = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, x, mean)
    call("anode_gpu_batch_var_3d1_packed_f32", S, C, N, 1e-5, x, mean, var)
    m1, v1 = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    call("anode_gpu_batch_mean_var_3d1_packed_f32", S, C, N, 1e-5, x, m1, v1)
    y = torch.empty(n, device="cuda")
    call("anode_gpu_batch_norm_3d1_packed_f32", S, C, N, x, mean, var, y)
    torch.cuda.synchronize()
    xv, yv = x.view(N, C, S), y.view(N, C, S)
    for c in (0, 1, 1023, 2046, 2047):
        col = xv[:, c, :].double()
        m = col.mean().item()
        v = ((col - float(mean[c])) ** 2).mean().item() + 1e-5
        assert abs(float(mean[c]) - m) <= 1e-5 * abs(m) + 1e-7
        assert abs(float(var[c]) - v) <= 1e-5 * v
        assert abs(float(m1[c]) - m) <= 1e-5 * abs(m) + 1e-7 and abs(float(v1[c]) - v) <= 1e-5 * v
        want = (xv[:, c, :] - mean[c]) / torch.sqrt(var[c])      # the map's own fp32 formula
        assert bool(((yv[:, c, :] - want).abs() <= 2e-6 * want.abs() + 1e-7).all())
        del col, want
    # the last sample (the far end of the array) on its own, every channel
    want = (xv[N - 1] - mean.view(C, 1)) / torch.sqrt(var.view(C, 1))
    assert bool(((yv[N - 1] - want).abs() <= 2e-6 * want.abs() + 1e-7).all())
    del y


def test_row_softmax_head_beyond_2_31(big):
    K, R = 1000, 2148000                 # 2 148 000 000 elements; rows in registers, one wave per row
    n = K * R
    assert (1 << 31) < n <= N_BIG
    x = big[:n]
    lab = torch.randint(0, K, (R,), device="cuda", dtype=torch.int32)
    dy = torch.full((R,), 0.5, device="cuda")
    p, nll, dx = torch.empty(n, device="cuda"), torch.empty(R, device="cuda"), torch.empty(n, device="cuda")
    call("anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32", K, R, x, lab, dy, p, nll, dx)
    idx = torch.empty(R, device="cuda", dtype=torch.int32)
    call("anode_gpu_arg_max_packed_u32", K, R, x, idx)
    torch.cuda.synchronize()
    pv, xv, dv = p.view(R, K), x.view(R, K), dx.view(R, K)
    for lo in (0, (1 << 31) // K - 500, R - 1000):     # the first rows, rows across 2^31, the last rows
        rows = slice(lo, lo + 1000)
        ref = torch.softmax(xv[rows].double(), dim=1)
        assert bool(((pv[rows].double() - ref).abs() <= 1e-5 * ref).all())
        picked = torch.gather(pv[rows], 1, lab[rows].long().unsqueeze(1)).squeeze(1)
        assert torch.allclose(nll[rows], -torch.log(picked), rtol=1e-5, atol=1e-6)
        onehot = torch.nn.functional.one_hot(lab[rows].long(), K).float()
        assert torch.equal(dv[rows], 0.5 * (pv[rows] - onehot))
        top = torch.gather(xv[rows], 1, idx[rows].long().unsqueeze(1)).squeeze(1)
        assert torch.equal(top, xv[rows].max(dim=1).values)
    sums = pv.sum(dim=1)
    assert bool(((sums - 1).abs() < 1e-5).all())
    del p, dx, sums


def test_long_odd_rows_beyond_2_31(big):
    # rows of 50 257 classes start anywhere in a 16-byte group: the streaming kernel over the array's aligned groups
    K, R = 50257, 42750                  # 2 148 486 750 elements
    n = K * R
    assert (1 << 31) < n <= N_BIG
    x = big[:n]
    lab = torch.randint(0, K, (R,), device="cuda", dtype=torch.int32)
    dy = torch.full((R,), 0.25, device="cuda")
    p, nll, dx = torch.empty(n, device="cuda"), torch.empty(R, device="cuda"), torch.empty(n, device="cuda")
    call("anode_gpu_softmax_cat_nll_fused_fwd_bwd_packed_f32", K, R, x, lab, dy, p, nll, dx)
    torch.cuda.synchronize()
    pv, xv, dv = p.view(R, K), x.view(R, K), dx.view(R, K)
    for lo in (0, (1 << 31) // K - 10, R - 20):        # the first rows, rows across 2^31, the last rows
        rows = slice(lo, lo + 20)
        ref = torch.softmax(xv[rows].double(), dim=1)
        assert bool(((pv[rows].double() - ref).abs() <= 1e-5 * ref).all())
        picked = torch.gather(pv[rows], 1, lab[rows].long().unsqueeze(1)).squeeze(1)
        assert torch.allclose(nll[rows], -torch.log(picked), rtol=1e-5, atol=1e-6)
        onehot = torch.nn.functional.one_hot(lab[rows].long(), K).float()
        assert torch.equal(dv[rows], 0.25 * (pv[rows] - onehot))
    sums = pv.sum(dim=1)
    assert bool(((sums - 1).abs() < 1e-5).all())
    del p, dx, sums


def test_casts_beyond_2_31(big):
    # quantize(dequantize(q)) == q for every code, and upcast is exact: 2^31 + 2^20 + 7 bytes in, 16-byte and tail paths
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    q = torch.randint(0, 256, (N_BIG,), device="cuda", dtype=torch.uint8, generator=g)
    f = torch.empty(N_BIG, device="cuda")
    call("anode_gpu_dequantize_u8_packed_f32", N_BIG, -1.0, 3.0, q, f)
    back = torch.empty(N_BIG, device="cuda", dtype=torch.uint8)
    call("anode_gpu_quantize_u8_packed_f32", N_BIG, -1.0, 3.0, f, back)
    torch.cuda.synchronize()
    assert torch.equal(back, q)
    assert float(f.min()) == -1.0 and abs(float(f.max()) - 3.0) <= 3e-7   # code 255: fma(255, fl(4/255), -1), one rounding
    del back
    u = f.view(torch.int32)              # reuse the 8.6 GB buffer
    call("anode_gpu_upcast_u8_packed_u32", N_BIG, q, u)
    torch.cuda.synchronize()
    step = 1 << 28
    for lo in range(0, N_BIG, step):
        hi = min(N_BIG, lo + step)
        assert torch.equal(u[lo:hi], q[lo:hi].to(torch.int32))
    del q, f, u


# ---- close to the largest array the 32-bit counts of the ABI can describe: 2^32 - 3 elements (17 GB) ----

N_MAX = (1 << 32) - 3


@pytest.fixture(scope="module")
def huge():
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    x = torch.empty(N_MAX + 4, device="cuda")
    x.normal_(generator=g)
    yield x
    del x
    torch.cuda.empty_cache()


@pytest.mark.parametrize("offset", [0, 1])
def test_flat_map_and_accumulate_close_to_2_32(huge, offset):
    x = huge[offset:offset + N_MAX]
    y = torch.full((N_MAX + 4,), float("nan"), device="cuda")
    call("anode_gpu_positive_clip_flat_map_f32", N_MAX, x, y[offset:offset + N_MAX])
    torch.cuda.synchronize()
    want = torch.relu(x)
    assert torch.equal(y[offset:offset + N_MAX], want)
    assert bool(torch.isnan(y[offset + N_MAX:]).all()) and bool(torch.isnan(y[:offset]).all())
    call("anode_gpu_add_packed_f32", N_MAX, x, y[offset:offset + N_MAX])   # y = relu(x) + x, applied exactly once
    torch.cuda.synchronize()
    want += x
    assert torch.equal(y[offset:offset + N_MAX], want)
    del y, want


def test_batch_norm_pieces_close_to_2_32(huge):
    S, C, N = 1 << 20, 3, 1365           # 4 293 918 720 elements
    n = S * C * N
    assert n < (1 << 32) and n > N_MAX - (1 << 21)
    x = huge[:n]
    mean, var = torch.empty(C, device="cuda"), torch.empty(C, device="cuda")
    call("anode_gpu_batch_mean_3d1_packed_f32", S, C, N, x, mean)
    call("anode_gpu_batch_var_3d1_packed_f32", S, C, N, 1e-5, x, mean, var)
    y = torch.empty(n, device="cuda")
    call("anode_gpu_batch_norm_3d1_packed_f32", S, C, N, x, mean, var, y)
    torch.cuda.synchronize()
    xv, yv = x.view(N, C, S), y.view(N, C, S)
    for c in range(C):
        m = xv[:, c, :].mean(dtype=torch.float64).item()
        v = xv[:, c, :].var(unbiased=False).item() + 1e-5
        assert abs(float(mean[c]) - m) <= 1e-5 * abs(m) + 1e-7
        assert abs(float(var[c]) - v) <= 2e-5 * v        # torch's own fp32 variance is the looser side here
        ym = yv[:, c, :].mean(dtype=torch.float64).item()
        yq = (yv[:, c, :].double() ** 2).mean().item() if c == C - 1 else None
        assert abs(ym) < 1e-4
        if yq is not None:                                 # the last channel ends at the last element of the array
            assert abs(yq - (1 - 1e-5 / v)) < 1e-4
    del y


def test_softmax_nd_backward_over_odd_planes_close_to_2_32(huge):
    # 4 294 574 085 elements in planes of 65535 pixels: the flat walk's last 16-byte group is a partial one, 2.7 * 10^5
    # elements under 2^32
    P, C, N = 65535, 19, 3449
    n = P * C * N
    assert (1 << 32) - (1 << 20) < n < (1 << 32) and n % 4 != 0
    p = huge[:n]
    lab = torch.randint(0, C, (P * N,), device="cuda", dtype=torch.int32)
    dy = torch.randn(P * N, device="cuda")
    dx = torch.empty(n + 8, device="cuda")
    dx[n:] = 555.0
    call("anode_gpu_softmax_nd_cat_nll_bwd_packed_f32", P, C, N, dy, p, lab, dx[:n])
    torch.cuda.synchronize()
    assert bool((dx[n:] == 555.0).all())
    pv, dv = p.view(N, C, P), dx[:n].view(N, C, P)
    ks = torch.arange(C, device="cuda", dtype=torch.int32).view(C, 1)
    for i in (0, N // 2, N - 1):
        want = dy.view(N, P)[i].unsqueeze(0) * (pv[i] - (lab.view(N, P)[i].unsqueeze(0) == ks).float())
        assert torch.equal(dv[i], want), i
    del dx, lab, dy


def test_softmax_nd_close_to_2_32(huge):
    P, C, N = 1 << 16, 19, 3449          # 4 294 639 616 elements
    n = P * C * N
    assert n < (1 << 32)
    x = huge[:n]
    p = torch.empty(n, device="cuda")
    call("anode_gpu_softmax_nd_packed_f32", P, C, N, x, p)
    torch.cuda.synchronize()
    pv = p.view(N, C, P)
    for i in (0, N // 2, N - 1):
        ref = torch.softmax(x.view(N, C, P)[i].double(), dim=0)
        assert bool(((pv[i].double() - ref).abs() <= 1e-5 * ref).all())
    sums = pv.sum(dim=1)
    assert bool(((sums - 1).abs() < 1e-5).all())
    del p, sums
