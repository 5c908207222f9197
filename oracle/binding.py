"""numpy binding of the CPU oracle (oracle/anode_oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
benchmark's CPU-baseline leg, never by the product package.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIBRARY_PATH = os.path.join(_HERE, "libanode_oracle.so")

DEFAULT_BLOCK = 1024  # tile width of the reference-order fp32 reductions

u32 = ctypes.c_uint32
f32 = ctypes.c_float
ptr = ctypes.c_void_p
cint = ctypes.c_int

MAP_OPS = {
    "copy": 0, "modulus": 1, "square": 2, "sqrt": 3, "positive_clip": 4, "logistic": 5,
    "unit_step": 6, "normal_cdf": 7, "tanh": 8, "rcosh2": 9, "leaky_relu": 10,
    "log_positive_clip": 11, "positive_reciprocal": 12,
}
MAP2_OPS = {"positive_clip_bwd": 0, "logistic_bwd": 1, "leaky_relu_bwd": 2, "copy_unit_step_join": 3}


def build(force: bool = False) -> str:
    if force or not os.path.exists(LIBRARY_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True, capture_output=True)
    return LIBRARY_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = ctypes.CDLL(build())
        _lib.oracle_arg_max.restype = ctypes.c_uint64
        _lib.oracle_arg_max.argtypes = [ptr, ctypes.c_uint64]
        _lib.oracle_max_threads.restype = cint
    return _lib


def _p(a):
    if a is None:
        return ptr(0)
    assert isinstance(a, np.ndarray) and a.flags["C_CONTIGUOUS"], "oracle takes contiguous numpy arrays"
    return ptr(a.ctypes.data)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _u32(a):
    return np.ascontiguousarray(a, dtype=np.uint32)


def max_threads() -> int:
    return int(lib().oracle_max_threads())


def set_threads(n: int) -> None:
    lib().oracle_set_threads(cint(n))


# --------------------------------------------------------------------------
# batch norm.  Arrays are flat, element (i0,i1,i2) at i0 + d0*(i1 + d1*i2).
# --------------------------------------------------------------------------

def batch_mean(d0, d1, d2, x, f64=False, bs=DEFAULT_BLOCK):
    x = _f32(x)
    if f64:
        out = np.empty(d1, np.float64)
        lib().oracle_batch_mean_f64(u32(d0), u32(d1), u32(d2), _p(x), _p(out))
    else:
        out = np.empty(d1, np.float32)
        lib().oracle_batch_mean_f32ref(u32(d0), u32(d1), u32(d2), _p(x), _p(out), u32(bs))
    return out


def batch_mean_bwd(d0, d1, d2, dmean, dx_in=None, f64=False):
    dmean = _f32(dmean)
    acc = dx_in is not None
    dx_in = _f32(dx_in) if acc else None
    n = d0 * d1 * d2
    if f64:
        out = np.empty(n, np.float64)
        lib().oracle_batch_mean_bwd_f64(u32(d0), u32(d1), u32(d2), _p(dmean), _p(dx_in),
                                        _p(out), cint(acc))
    else:
        out = dx_in.copy() if acc else np.empty(n, np.float32)
        lib().oracle_batch_mean_bwd_f32ref(u32(d0), u32(d1), u32(d2), _p(dmean), _p(out), cint(acc))
    return out


def batch_var(d0, d1, d2, eps, x, mean, f64=False, bs=DEFAULT_BLOCK):
    x, mean = _f32(x), _f32(mean)
    if f64:
        out = np.empty(d1, np.float64)
        lib().oracle_batch_var_f64(u32(d0), u32(d1), u32(d2), f32(eps), _p(x), _p(mean), _p(out))
    else:
        out = np.empty(d1, np.float32)
        lib().oracle_batch_var_f32ref(u32(d0), u32(d1), u32(d2), f32(eps), _p(x), _p(mean), _p(out), u32(bs))
    return out


def batch_var_bwd(d0, d1, d2, dvar, x, mean, dx_in=None, f64=False):
    dvar, x, mean = _f32(dvar), _f32(x), _f32(mean)
    acc = dx_in is not None
    dx_in = _f32(dx_in) if acc else None
    n = d0 * d1 * d2
    if f64:
        out = np.empty(n, np.float64)
        lib().oracle_batch_var_bwd_f64(u32(d0), u32(d1), u32(d2), _p(dvar), _p(x), _p(mean),
                                       _p(dx_in), _p(out), cint(acc))
    else:
        out = dx_in.copy() if acc else np.empty(n, np.float32)
        lib().oracle_batch_var_bwd_f32ref(u32(d0), u32(d1), u32(d2), _p(dvar), _p(x), _p(mean), _p(out), cint(acc))
    return out


def batch_var_bwd_mean(d0, d1, d2, dvar, x, mean, dmean_in=None, f64=False, bs=DEFAULT_BLOCK):
    dvar, x, mean = _f32(dvar), _f32(x), _f32(mean)
    acc = dmean_in is not None
    dmean_in = _f32(dmean_in) if acc else None
    if f64:
        out = np.empty(d1, np.float64)
        lib().oracle_batch_var_bwd_mean_f64(u32(d0), u32(d1), u32(d2), _p(dvar), _p(x), _p(mean),
                                            _p(dmean_in), _p(out), cint(acc))
    else:
        out = dmean_in.copy() if acc else np.empty(d1, np.float32)
        lib().oracle_batch_var_bwd_mean_f32ref(u32(d0), u32(d1), u32(d2), _p(dvar), _p(x), _p(mean), _p(out),
                                               cint(acc), u32(bs))
    return out


def batch_norm(d0, d1, d2, x, mean, var, f64=False):
    x, mean, var = _f32(x), _f32(mean), _f32(var)
    out = np.empty(d0 * d1 * d2, np.float64 if f64 else np.float32)
    fn = lib().oracle_batch_norm_f64 if f64 else lib().oracle_batch_norm_f32ref
    fn(u32(d0), u32(d1), u32(d2), _p(x), _p(mean), _p(var), _p(out))
    return out


def batch_norm_bwd(d0, d1, d2, dy, var, dx_in=None, f64=False):
    dy, var = _f32(dy), _f32(var)
    acc = dx_in is not None
    dx_in = _f32(dx_in) if acc else None
    n = d0 * d1 * d2
    if f64:
        out = np.empty(n, np.float64)
        lib().oracle_batch_norm_bwd_f64(u32(d0), u32(d1), u32(d2), _p(dy), _p(var),
                                        _p(dx_in), _p(out), cint(acc))
    else:
        out = dx_in.copy() if acc else np.empty(n, np.float32)
        lib().oracle_batch_norm_bwd_f32ref(u32(d0), u32(d1), u32(d2), _p(dy), _p(var), _p(out), cint(acc))
    return out


def batch_norm_bwd_mean(d0, d1, d2, dy, var, dmean_in=None, f64=False, bs=DEFAULT_BLOCK):
    dy, var = _f32(dy), _f32(var)
    acc = dmean_in is not None
    dmean_in = _f32(dmean_in) if acc else None
    if f64:
        out = np.empty(d1, np.float64)
        lib().oracle_batch_norm_bwd_mean_f64(u32(d0), u32(d1), u32(d2), _p(dy), _p(var),
                                             _p(dmean_in), _p(out), cint(acc))
    else:
        out = dmean_in.copy() if acc else np.empty(d1, np.float32)
        lib().oracle_batch_norm_bwd_mean_f32ref(u32(d0), u32(d1), u32(d2), _p(dy), _p(var), _p(out), cint(acc), u32(bs))
    return out


def batch_norm_bwd_var(d0, d1, d2, dy, x, mean, var, dvar_in=None, f64=False, bs=DEFAULT_BLOCK):
    dy, x, mean, var = _f32(dy), _f32(x), _f32(mean), _f32(var)
    acc = dvar_in is not None
    dvar_in = _f32(dvar_in) if acc else None
    if f64:
        out = np.empty(d1, np.float64)
        lib().oracle_batch_norm_bwd_var_f64(u32(d0), u32(d1), u32(d2), _p(dy), _p(x), _p(mean), _p(var),
                                            _p(dvar_in), _p(out), cint(acc))
    else:
        out = dvar_in.copy() if acc else np.empty(d1, np.float32)
        lib().oracle_batch_norm_bwd_var_f32ref(u32(d0), u32(d1), u32(d2), _p(dy), _p(x), _p(mean), _p(var), _p(out),
                                               cint(acc), u32(bs))
    return out


def batch_norm_bwd_var_v2(d0, d1, d2, dy, y, var, dvar_in=None, f64=False, bs=DEFAULT_BLOCK):
    dy, y, var = _f32(dy), _f32(y), _f32(var)
    acc = dvar_in is not None
    dvar_in = _f32(dvar_in) if acc else None
    if f64:
        out = np.empty(d1, np.float64)
        lib().oracle_batch_norm_bwd_var_v2_f64(u32(d0), u32(d1), u32(d2), _p(dy), _p(y), _p(var),
                                               _p(dvar_in), _p(out), cint(acc))
    else:
        out = dvar_in.copy() if acc else np.empty(d1, np.float32)
        lib().oracle_batch_norm_bwd_var_v2_f32ref(u32(d0), u32(d1), u32(d2), _p(dy), _p(y), _p(var), _p(out),
                                                  cint(acc), u32(bs))
    return out


# --------------------------------------------------------------------------
# softmax / NLL
# --------------------------------------------------------------------------

def softmax(d0, d1, x, f64=False, bs=DEFAULT_BLOCK):
    x = _f32(x)
    if f64:
        out = np.empty(d0 * d1, np.float64)
        lib().oracle_softmax_f64(u32(d0), u32(d1), _p(x), _p(out))
    else:
        out = np.empty(d0 * d1, np.float32)
        lib().oracle_softmax_f32ref(u32(d0), u32(d1), _p(x), _p(out), u32(bs))
    return out


def softmax_cat_nll(d0, d1, p, cat, f64=False):
    p, cat = _f32(p), _u32(cat)
    out = np.empty(d1, np.float64 if f64 else np.float32)
    fn = lib().oracle_softmax_cat_nll_f64 if f64 else lib().oracle_softmax_cat_nll_f32ref
    fn(u32(d0), u32(d1), _p(p), _p(cat), _p(out))
    return out


def softmax_cat_gather_index(d0, d1, cat):
    cat = _u32(cat)
    out = np.empty(d1, np.uint64)
    lib().oracle_softmax_cat_gather_index(u32(d0), u32(d1), _p(cat), _p(out))
    return out


def softmax_cat_nll_bwd(d0, d1, dy, p, cat, dx_in=None, f64=False):
    dy, p, cat = _f32(dy), _f32(p), _u32(cat)
    acc = dx_in is not None
    dx_in = _f32(dx_in) if acc else None
    if f64:
        out = np.empty(d0 * d1, np.float64)
        lib().oracle_softmax_cat_nll_bwd_f64(u32(d0), u32(d1), _p(dy), _p(p), _p(cat),
                                             _p(dx_in), _p(out), cint(acc))
    else:
        out = dx_in.copy() if acc else np.empty(d0 * d1, np.float32)
        lib().oracle_softmax_cat_nll_bwd_f32ref(u32(d0), u32(d1), _p(dy), _p(p), _p(cat), _p(out), cint(acc))
    return out


def softmax_nd(P, C, N, x, f64=False):
    x = _f32(x)
    out = np.empty(P * C * N, np.float64 if f64 else np.float32)
    fn = lib().oracle_softmax_nd_f64 if f64 else lib().oracle_softmax_nd_f32ref
    fn(u32(P), u32(C), u32(N), _p(x), _p(out))
    return out


def softmax_nd_cat_nll(P, C, N, p, cat, f64=False):
    p, cat = _f32(p), _u32(cat)
    out = np.empty(P * N, np.float64 if f64 else np.float32)
    fn = lib().oracle_softmax_nd_cat_nll_f64 if f64 else lib().oracle_softmax_nd_cat_nll_f32ref
    fn(u32(P), u32(C), u32(N), _p(p), _p(cat), _p(out))
    return out


def softmax_nd_cat_gather_index(P, C, N, cat):
    cat = _u32(cat)
    out = np.empty(P * N, np.uint64)
    lib().oracle_softmax_nd_cat_gather_index(u32(P), u32(C), u32(N), _p(cat), _p(out))
    return out


def softmax_nd_cat_nll_bwd(P, C, N, dy, p, cat, dx_in=None, f64=False):
    dy, p, cat = _f32(dy), _f32(p), _u32(cat)
    acc = dx_in is not None
    dx_in = _f32(dx_in) if acc else None
    if f64:
        out = np.empty(P * C * N, np.float64)
        lib().oracle_softmax_nd_cat_nll_bwd_f64(u32(P), u32(C), u32(N), _p(dy), _p(p), _p(cat),
                                                _p(dx_in), _p(out), cint(acc))
    else:
        out = dx_in.copy() if acc else np.empty(P * C * N, np.float32)
        lib().oracle_softmax_nd_cat_nll_bwd_f32ref(u32(P), u32(C), u32(N), _p(dy), _p(p), _p(cat), _p(out), cint(acc))
    return out


# --------------------------------------------------------------------------
# flat maps, casts, discrete, F1, argmax
# --------------------------------------------------------------------------

def flat_map(op, x, c=0.0, f64=False):
    x = _f32(x).ravel()
    out = np.empty(x.size, np.float64 if f64 else np.float32)
    fn = lib().oracle_flat_map_f64 if f64 else lib().oracle_flat_map_f32ref
    rc = fn(cint(MAP_OPS[op]), u32(x.size), f32(c), _p(x), _p(out))
    assert rc == 0
    return out


def flat_map2(op, a, b, c=0.0):
    a, b = _f32(a).ravel(), _f32(b).ravel()
    out = np.empty(a.size, np.float32)
    rc = lib().oracle_flat_map2_f32ref(cint(MAP2_OPS[op]), u32(a.size), f32(c), _p(a), _p(b), _p(out))
    assert rc == 0
    return out


def upcast_u8(x):
    x = np.ascontiguousarray(x, dtype=np.uint8).ravel()
    out = np.empty(x.size, np.uint32)
    lib().oracle_upcast_u8_u32(u32(x.size), _p(x), _p(out))
    return out


def dequantize_u8(lo, hi, x, fused=True):
    x = np.ascontiguousarray(x, dtype=np.uint8).ravel()
    out = np.empty(x.size, np.float32)
    fn = lib().oracle_dequantize_u8_f32ref if fused else lib().oracle_dequantize_u8_f32_unfused
    fn(u32(x.size), f32(lo), f32(hi), _p(x), _p(out))
    return out


def one_hot(d0, K, d2, cat):
    cat = _u32(cat)
    out = np.empty(d0 * K * d2, np.float32)
    lib().oracle_discrete_one_hot(u32(d0), u32(K), u32(d2), _p(cat), _p(out))
    return out


def f1_loss(d0, K, d2, eps, x, target, f64=False, bs=DEFAULT_BLOCK):
    x, target = _f32(x), _f32(target)
    if f64:
        out = np.empty(K * d2, np.float64)
        lib().oracle_smooth_negative_f1_loss_f64(u32(d0), u32(K), u32(d2), f32(eps), _p(x), _p(target), _p(out))
    else:
        out = np.empty(K * d2, np.float32)
        lib().oracle_smooth_negative_f1_loss_f32ref(u32(d0), u32(K), u32(d2), f32(eps), _p(x), _p(target), _p(out),
                                                    u32(bs))
    return out


def f1_loss_bwd(d0, K, d2, eps, dy, x, target, f64=False):
    dy, x, target = _f32(dy), _f32(x), _f32(target)
    out = np.empty(d0 * K * d2, np.float64 if f64 else np.float32)
    fn = lib().oracle_smooth_negative_f1_loss_bwd_f64 if f64 else lib().oracle_smooth_negative_f1_loss_bwd_f32ref
    fn(u32(d0), u32(K), u32(d2), f32(eps), _p(dy), _p(x), _p(target), _p(out))
    return out


def arg_max(xs) -> int:
    xs = _f32(xs).ravel()
    return int(lib().oracle_arg_max(_p(xs), ctypes.c_uint64(xs.size)))


def arg_max_rows(d0, d1, x):
    x = _f32(x)
    out = np.empty(d1, np.uint32)
    lib().oracle_arg_max_rows(u32(d0), u32(d1), _p(x), _p(out))
    return out


# --------------------------------------------------------------------------
# additive symbols (no kernel in the reference)
# --------------------------------------------------------------------------

def quantize_u8(lo, hi, x):
    x = _f32(x).ravel()
    out = np.empty(x.size, np.uint8)
    lib().oracle_quantize_u8(u32(x.size), f32(lo), f32(hi), _p(x), _p(out))
    return out


def bcast_flat_mult_add(inner, bcast, outer, lx, rx, shift=None):
    lx, rx = _f32(lx), _f32(rx)
    out = np.empty(inner * bcast * outer, np.float32)
    shift = _f32(shift) if shift is not None else None
    lib().oracle_bcast_flat_mult_add(u32(inner), u32(bcast), u32(outer), _p(lx), _p(rx), _p(shift), _p(out))
    return out


def bcast_dequantize_u8(inner, bcast, outer, a, b, q):
    a, b = _f32(a), _f32(b)
    q = np.ascontiguousarray(q, dtype=np.uint8).ravel()
    out = np.empty(inner * bcast * outer, np.float32)
    lib().oracle_bcast_dequantize_u8(u32(inner), u32(bcast), u32(outer), _p(a), _p(b), _p(q), _p(out))
    return out


def batch_mean_var(d0, d1, d2, eps, x):
    x = _f32(x)
    mean = np.empty(d1, np.float64)
    var = np.empty(d1, np.float64)
    lib().oracle_batch_mean_var_f64(u32(d0), u32(d1), u32(d2), f32(eps), _p(x), _p(mean), _p(var))
    return mean, var


def online_average(rate, x, y):
    x = _f32(x).ravel()
    out = _f32(y).ravel().copy()
    lib().oracle_online_average(u32(x.size), f32(rate), _p(x), _p(out))
    return out


def channel_sum(d0, d1, d2, x, square=False):
    x = _f32(x)
    out = np.empty(d1, np.float64)
    lib().oracle_channel_sum_f64(u32(d0), u32(d1), u32(d2), cint(int(square)), _p(x), _p(out))
    return out


def batch_norm_affine(d0, d1, d2, x, mean, var, gamma, beta, f64=False):
    x, mean, var, gamma, beta = _f32(x), _f32(mean), _f32(var), _f32(gamma), _f32(beta)
    out = np.empty(d0 * d1 * d2, np.float64 if f64 else np.float32)
    fn = lib().oracle_batch_norm_affine_f64 if f64 else lib().oracle_batch_norm_affine_f32ref
    fn(u32(d0), u32(d1), u32(d2), _p(x), _p(mean), _p(var), _p(gamma), _p(beta), _p(out))
    return out


# --------------------------------------------------------------------------
# neighbours from gpudevicemem (closed forms of the call sites)
# --------------------------------------------------------------------------

def sum_packed(x) -> float:
    x = _f32(x).ravel()
    fn = lib().oracle_sum_packed_f64
    fn.restype = ctypes.c_double
    return float(fn(u32(x.size), _p(x)))


def online_discount(rate, x, y):
    x = _f32(x).ravel()
    out = _f32(y).ravel().copy()
    lib().oracle_online_discount(u32(x.size), f32(rate), _p(x), _p(out))
    return out


def online_add(rate, x, y):
    x = _f32(x).ravel()
    out = _f32(y).ravel().copy()
    lib().oracle_online_add(u32(x.size), f32(rate), _p(x), _p(out))
    return out


def flat_bcast_rdiv(inner, outer, x, r):
    x, r = _f32(x).ravel(), _f32(r).ravel()
    out = np.empty(inner * outer, np.float32)
    lib().oracle_flat_bcast_rdiv(u32(inner), u32(outer), _p(x), _p(r), _p(out))
    return out
