"""Helpers shared by the GPU parity tests: device buffers, calls through the
C ABI and the comparison bars.

Bars:
  * bit-exact for integer / byte / index work and for maps whose fp32
    arithmetic is fully specified (compare, multiply, correctly rounded
    divide and sqrt, the fused multiply-adds the reference's compiler forms);
  * |got - ref| <= 1e-5 * |ref| (+ a stated absolute floor) against the fp64
    oracle for batch-norm and softmax.
"""
import numpy as np
import torch

from anode_amd import gpu
from anode_amd._lib import KernelConfig

F32 = np.float32
REL = 1e-5  # the relative bar for the tolerance class


def dev(a, offset=0):
    """Upload a numpy array.  offset > 0 places it `offset` elements into a larger
    allocation, so the device pointer is only element-aligned (views in anode
    can start at any element: as_dptr() on a view)."""
    a = np.ascontiguousarray(a)
    t = torch.from_numpy(a.ravel())
    if offset == 0:
        return t.cuda()
    buf = torch.empty(a.size + offset + 8, dtype=t.dtype, device="cuda")
    view = buf[offset:offset + a.size]
    view.copy_(t)
    return view


def empty(n, dtype=torch.float32, offset=0, fill=None):
    buf = torch.empty(n + offset + 8, dtype=dtype, device="cuda")
    if fill is None:
        # poison so that elements the kernel fails to write are noticed
        if dtype == torch.float32:
            buf.fill_(float("nan"))
        else:
            buf.fill_(123)
    else:
        buf.fill_(fill)
    return buf[offset:offset + n]


def host(t):
    torch.cuda.synchronize()
    return t.detach().cpu().numpy()


def call(name, *args, **kw):
    gpu.call(name, *args, **kw)
    err = gpu.take_last_error()
    assert err == 0, f"{name}: launch error {err}"


def bits(a):
    a = np.ascontiguousarray(a)
    return a.view(np.uint32) if a.dtype == np.float32 else a


def assert_bit_exact(got, want, what=""):
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if got.dtype == np.float32:
        nan_g, nan_w = np.isnan(got), np.isnan(want)
        assert np.array_equal(nan_g, nan_w), f"{what}: NaN pattern differs"
        ok = ~nan_w
        same = bits(got)[ok] == bits(want)[ok]
    else:
        same = got == want
    if not np.all(same):
        bad = np.flatnonzero(~same)
        i = bad[0]
        raise AssertionError(f"{what}: {bad.size} of {same.size} elements differ; first at {i}: "
                             f"got {got[ok][i] if got.dtype == np.float32 else got[i]!r} "
                             f"want {want[ok][i] if got.dtype == np.float32 else want[i]!r}")


def rms(a):
    a = np.asarray(a, np.float64)
    a = a[np.isfinite(a)]
    return float(np.sqrt(np.mean(a * a))) if a.size else 0.0


def assert_close(got, ref64, what="", rel=REL, abs_floor=0.0):
    """|got - ref| <= rel*|ref| + abs_floor; NaNs must coincide, infinities must be equal."""
    got = np.asarray(got, np.float64)
    ref64 = np.asarray(ref64, np.float64)
    assert got.shape == ref64.shape, (what, got.shape, ref64.shape)
    nan_g, nan_r = np.isnan(got), np.isnan(ref64)
    assert np.array_equal(nan_g, nan_r), f"{what}: NaN pattern differs ({nan_g.sum()} vs {nan_r.sum()})"
    ok = ~nan_r
    inf_r = np.isinf(ref64)
    assert np.array_equal(got[inf_r], ref64[inf_r]), f"{what}: infinities differ"
    ok &= ~inf_r
    err = np.abs(got[ok] - ref64[ok])
    bound = rel * np.abs(ref64[ok]) + abs_floor
    if not np.all(err <= bound):
        i = int(np.argmax(err - bound))
        raise AssertionError(f"{what}: {(err > bound).sum()} of {err.size} outside the bar; worst: got {got[ok][i]!r} "
                             f"ref {ref64[ok][i]!r} err {err[i]:.3e} bound {bound[i]:.3e}")


def cfg(block=1024, max_blocks=1024):
    return KernelConfig(block, max_blocks)
