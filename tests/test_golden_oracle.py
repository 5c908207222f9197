"""The committed fixtures under tests/golden/ against the CPU oracle.

small_cases.npz was written by tests/golden/make_golden.py from the oracle; re-deriving it here keeps an edit to
the oracle (or a different libm) from drifting unnoticed.  reference_known_answers.json holds the values the
reference's own tests assert (tests/test_gpu.rs:561-758); the oracle has to reproduce them.
"""
import json
import os

import numpy as np
import pytest

from oracle import binding as O

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN = os.path.join(HERE, "golden")
F32 = np.float32

# results that go through expf/logf/tanhf/erff of the host libm: equal to 2 ulp, everything else to the bit
LIBM_KEYS = ("/p", "/nll", "/dx", "logistic", "normal_cdf", "tanh", "rcosh2", "log_positive_clip")


def _same(a, b, exact):
    a, b = np.asarray(a), np.asarray(b)
    assert a.shape == b.shape and a.dtype == b.dtype
    nan = np.isnan(a) if a.dtype.kind == "f" else np.zeros(a.shape, bool)
    assert np.array_equal(nan, np.isnan(b) if b.dtype.kind == "f" else nan)
    if exact or a.dtype.kind != "f":
        return np.array_equal(a[~nan].view(np.uint8), b[~nan].view(np.uint8))
    with np.errstate(invalid="ignore"):
        return bool(np.all((a[~nan] == b[~nan]) | (np.abs(a[~nan] - b[~nan]) <= 2 * np.spacing(np.abs(b[~nan])))))


def test_small_cases_reproduce():
    import importlib.util
    spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    fresh = mod.cases()
    with np.load(os.path.join(GOLDEN, "small_cases.npz")) as stored:
        assert sorted(stored.files) == sorted(fresh)
        for k in stored.files:
            libm = any(t in k for t in LIBM_KEYS) and not k.startswith(("bn_", "cast", "one_hot", "flat2"))
            assert _same(fresh[k], stored[k], exact=not libm), k


@pytest.fixture(scope="module")
def known():
    with open(os.path.join(GOLDEN, "reference_known_answers.json")) as f:
        return json.load(f)


def test_known_softmax_zeros(known):
    k = known["softmax_zeros"]
    p = O.softmax(k["K"], k["rows"], np.full(k["K"] * k["rows"], k["logits_fill"], F32))
    assert np.all(p == F32(k["p_expected_each"]))


def test_known_softmax_cat_nll(known):
    k = known["softmax_cat_nll"]
    K, R = k["K"], k["rows"]
    p = O.softmax(K, R, np.full(K * R, k["logits_fill"], F32))
    assert np.all(p == F32(k["p_expected_each"]))
    nll = O.softmax_cat_nll(K, R, p, np.array(k["labels"], np.uint32))
    assert np.allclose(nll, k["nll_expected_each_f64"], rtol=k["nll_rel_tol"], atol=0)
    assert abs(k["nll_expected_each_f64"] - np.log(32.0)) < 1e-15


def test_known_out_of_range_label(known):
    k = known["softmax_cat_nll_out_of_range"]
    K, R = k["K"], k["rows"]
    p = O.softmax(K, R, np.zeros(K * R, F32))
    nll = O.softmax_cat_nll(K, R, p, np.array(k["labels"], np.uint32))
    assert list(np.isnan(nll)) == k["nll_is_nan"]
    assert bool(np.isnan(nll.sum())) == k["batch_sum_is_nan"]


def test_known_adjoint(known):
    k = known["softmax_cat_nll_adjoint"]
    K, R = k["K"], k["rows"]
    p = O.softmax(K, R, np.zeros(K * R, F32))
    labels = np.array(k["labels"], np.uint32)
    dx = O.softmax_cat_nll_bwd(K, R, np.full(R, k["dy_fill"], F32), p, labels).reshape(R, K)
    want = np.full((R, K), k["dx_expected_off_label"], F32)
    want[np.arange(R), labels] = k["dx_expected_on_label"]
    assert np.array_equal(dx, want)


def test_known_dequantize(known):
    k = known["dequantize_one"]
    y = O.dequantize_u8(k["lo"], k["hi"], np.full(k["count"], k["code"], np.uint8))
    assert np.all(y == F32(1.0) / F32(255.0))


def test_known_online_average(known):
    k = known["online_average"]
    x = np.full(k["count"], k["x_fill"], F32)
    y = np.full(k["count"], k["y_fill"], F32)
    y = O.online_average(k["rate"], x, y)
    assert np.all(y == F32(k["after_first"]))
    y = O.online_average(k["rate"], x, y)
    assert np.all(y == F32(k["after_second"]))
