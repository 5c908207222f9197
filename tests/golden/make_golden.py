"""Writes tests/golden/small_cases.npz: inputs and expected outputs of every reference entry point at small,
ragged shapes.

    python tests/golden/make_golden.py

The expected values come from the CPU oracle (fp32 flavour with the reference's operation order, plus the fp64
flavour for the tolerance-class results) after tests/test_oracle_pins.py has pinned it.  The file is data only; the
tests compare both the oracle (so that an edit to it cannot drift unnoticed) and the GPU library against it.
reference_known_answers.json beside it is written by hand from the reference's own tests (tests/test_gpu.rs:561-758)
and is not touched by this script.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import binding as O  # noqa: E402

F32 = np.float32

# (dim0, dim1, dim2) = (S, C, N): odd S, S = 1, S a multiple of 4, C = 1
BN_SHAPES = [(7, 3, 5), (49, 8, 4), (1, 5, 9), (64, 1, 3)]
ROW_SHAPES = [(10, 32), (1000, 3), (33, 7), (1, 4)]        # (K, rows)
ND_SHAPES = [(37, 19, 2), (8, 3, 1), (5, 70, 2)]            # (pixels, C, N)
EPS = 1e-5


def cases():
    g = np.random.default_rng(20181116)
    out = {}

    for S, C, N in BN_SHAPES:
        k = f"bn_{S}x{C}x{N}"
        d = (S, C, N)
        x = (2 + 3 * g.standard_normal(S * C * N)).astype(F32)
        dy = g.standard_normal(S * C * N).astype(F32)
        mean = O.batch_mean(*d, x)
        var = O.batch_var(*d, EPS, x, mean)
        y = O.batch_norm(*d, x, mean, var)
        dx1 = O.batch_norm_bwd(*d, dy, var)
        dmean1 = O.batch_norm_bwd_mean(*d, dy, var)
        dvar = O.batch_norm_bwd_var(*d, dy, x, mean, var)
        dvar_v2 = O.batch_norm_bwd_var_v2(*d, dy, y, var)
        dx2 = O.batch_var_bwd(*d, dvar, x, mean, dx_in=dx1)
        dmean2 = O.batch_var_bwd_mean(*d, dvar, x, mean, dmean_in=dmean1)
        dx3 = O.batch_mean_bwd(*d, dmean2, dx_in=dx2)
        out.update({f"{k}/x": x, f"{k}/dy": dy, f"{k}/mean": mean, f"{k}/var": var, f"{k}/y": y, f"{k}/dx1": dx1,
                    f"{k}/dmean1": dmean1, f"{k}/dvar": dvar, f"{k}/dvar_v2": dvar_v2, f"{k}/dx2": dx2,
                    f"{k}/dmean2": dmean2, f"{k}/dx3": dx3,
                    f"{k}/mean64": O.batch_mean(*d, x, f64=True), f"{k}/var64": O.batch_var(*d, EPS, x, mean, f64=True),
                    f"{k}/dvar64": O.batch_norm_bwd_var(*d, dy, x, mean, var, f64=True),
                    f"{k}/dmean1_64": O.batch_norm_bwd_mean(*d, dy, var, f64=True)})

    for K, R in ROW_SHAPES:
        k = f"row_{K}x{R}"
        x = (2 * g.standard_normal(K * R)).astype(F32)
        cat = g.integers(0, K, R).astype(np.uint32)
        cat[-1] = K + 3                                    # out of range: NaN loss, unmasked gradient
        dy = g.standard_normal(R).astype(F32)
        p = O.softmax(K, R, x)
        out.update({f"{k}/x": x, f"{k}/cat": cat, f"{k}/dy": dy, f"{k}/p": p, f"{k}/p64": O.softmax(K, R, x, f64=True),
                    f"{k}/nll": O.softmax_cat_nll(K, R, p, cat), f"{k}/nll64": O.softmax_cat_nll(K, R, p, cat, f64=True),
                    f"{k}/dx": O.softmax_cat_nll_bwd(K, R, dy, p, cat)})

    for P, C, N in ND_SHAPES:
        k = f"nd_{P}x{C}x{N}"
        x = g.standard_normal(P * C * N).astype(F32)
        cat = g.integers(0, C, P * N).astype(np.uint32)
        cat[::7] = 255
        dy = g.standard_normal(P * N).astype(F32)
        p = O.softmax_nd(P, C, N, x)
        out.update({f"{k}/x": x, f"{k}/cat": cat, f"{k}/dy": dy, f"{k}/p": p,
                    f"{k}/p64": O.softmax_nd(P, C, N, x, f64=True),
                    f"{k}/nll": O.softmax_nd_cat_nll(P, C, N, p, cat),
                    f"{k}/nll64": O.softmax_nd_cat_nll(P, C, N, p, cat, f64=True),
                    f"{k}/dx": O.softmax_nd_cat_nll_bwd(P, C, N, dy, p, cat)})

    q = g.integers(0, 256, 1001, dtype=np.uint8)
    q[:256] = np.arange(256, dtype=np.uint8)
    out["cast/q"] = q
    out["cast/upcast"] = O.upcast_u8(q)
    out["cast/dequantize_0_1"] = O.dequantize_u8(0.0, 1.0, q)
    out["cast/dequantize_m1p5_2p25"] = O.dequantize_u8(-1.5, 2.25, q)
    oh = g.integers(0, 9, 5 * 3).astype(np.uint32)            # classes 7, 8 are out of range for K = 7: all-zero columns
    out["one_hot/cat_5x7x3"] = oh
    out["one_hot/y_5x7x3"] = O.one_hot(5, 7, 3, oh)

    special = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-42, -1e-42, 3.5, -3.5, 88.0, -88.0], F32)
    fx = np.concatenate([special, (3 * g.standard_normal(257 - special.size)).astype(F32)])
    fb = g.standard_normal(257).astype(F32)
    out["flat/x"], out["flat/b"] = fx, fb
    for op in O.MAP_OPS:
        c = 0.125 if op == "leaky_relu" else 0.0
        with np.errstate(all="ignore"):
            out[f"flat/{op}"] = O.flat_map(op, fx, c)
            out[f"flat/{op}64"] = O.flat_map(op, fx, c, f64=True)
    for op in O.MAP2_OPS:
        out[f"flat2/{op}"] = O.flat_map2(op, fb, fx, 0.125 if op == "leaky_relu_bwd" else 0.0)

    S, K, N = 23, 4, 3
    fxp = g.random(S * K * N).astype(F32)
    ft = (g.random(S * K * N) < 0.3).astype(F32)
    fdy = g.standard_normal(K * N).astype(F32)
    out.update({"f1/x": fxp, "f1/target": ft, "f1/dy": fdy, "f1/loss": O.f1_loss(S, K, N, 1e-3, fxp, ft),
                "f1/loss64": O.f1_loss(S, K, N, 1e-3, fxp, ft, f64=True),
                "f1/dx": O.f1_loss_bwd(S, K, N, 1e-3, fdy, fxp, ft)})
    return out


if __name__ == "__main__":
    O.build()
    data = cases()
    path = os.path.join(HERE, "small_cases.npz")
    np.savez_compressed(path, **data)
    print(f"wrote {path}: {len(data)} arrays, {os.path.getsize(path)} bytes")
