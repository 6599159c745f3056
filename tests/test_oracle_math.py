"""include/ssr_math.h (host build, through the oracle library) against float64 libm."""
import numpy as np


def _ulp_err(got, want64):
    want32 = want64.astype(np.float32)
    ulp = np.spacing(np.abs(want32)).astype(np.float64)
    ulp = np.maximum(ulp, np.finfo(np.float32).tiny)
    return np.abs(got.astype(np.float64) - want64) / ulp


def test_exp(oracle):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.uniform(-87, 88, 200000), rng.uniform(-12, 3, 200000),
                        np.array([0.0, -0.0, 1.0, -1.0, 88.7, -87.29])]).astype(np.float32)
    err = _ulp_err(oracle.math(0, x), np.exp(x.astype(np.float64)))
    assert err.max() < 1.5, err.max()
    assert oracle.math(0, np.array([-87.31, -200, -np.inf], np.float32)).tolist() == [0, 0, 0]
    assert np.isinf(oracle.math(0, np.array([89.0], np.float32))[0])
    assert np.isnan(oracle.math(0, np.array([np.nan], np.float32))[0])
    assert oracle.math(0, np.array([0.0], np.float32))[0] == 1.0


def test_log(oracle):
    rng = np.random.default_rng(2)
    x = np.concatenate([np.exp(rng.uniform(-80, 80, 200000)), rng.uniform(0.5, 300, 200000),
                        np.array([1.0, 255.0, 1e-40, 3e-39])]).astype(np.float32)
    err = _ulp_err(oracle.math(1, x), np.log(x.astype(np.float64)))
    # near x = 1 the result is tiny; bound the absolute error there instead
    near1 = np.abs(x - 1) < 0.25
    assert err[~near1].max() < 1.5, err[~near1].max()
    assert np.abs(oracle.math(1, x)[near1] - np.log(x[near1].astype(np.float64))).max() < 6e-8
    out = oracle.math(1, np.array([0.0, -1.0, np.inf], np.float32))
    assert out[0] == -np.inf and np.isnan(out[1]) and out[2] == np.inf
    assert oracle.math(1, np.array([1.0], np.float32))[0] == 0.0


def test_atan2(oracle):
    rng = np.random.default_rng(3)
    y = rng.normal(0, 5, 400000).astype(np.float32)
    x = rng.normal(0, 5, 400000).astype(np.float32)
    got = oracle.math(2, y, x)
    want = np.arctan2(y.astype(np.float64), x.astype(np.float64))
    assert np.abs(got - want).max() < 4e-7
    # quadrants and axes
    yy = np.array([0, 1, -1, 0, 1, -1, 0], np.float32)
    xx = np.array([1, 0, 0, -1, -1, -1, 0], np.float32)
    got = oracle.math(2, yy, xx)
    want = np.array([0, np.pi / 2, -np.pi / 2, np.pi, 3 * np.pi / 4, -3 * np.pi / 4, 0])
    assert np.abs(got - want).max() < 3e-7


def test_sigmoid(oracle):
    x = np.linspace(-30, 30, 10001).astype(np.float32)
    got = oracle.math(3, x)
    want = 1 / (1 + np.exp(-x.astype(np.float64)))
    assert np.abs(got - want).max() < 1.5e-7


def test_adam_inverse_bias_corrections(oracle):
    """1 / (1 - beta^t) with the reference's FLOAT betas (FusedProjectionBwdOptim_kernel.cuh:369-370): against
    float64 powers of float32(0.9) / float32(0.999). The power is within 2 ulp, so the correction is within
    2 ulp of the power's spacing divided by (1 - beta^t) -- and nowhere near the 1.3e-5 by which a correction
    built on the double constant 0.999 is off at small t."""
    t = np.concatenate([np.arange(1, 3000), np.array([5000, 30000, 100000, 1000000])]).astype(np.float32)
    for op, beta in ((4, np.float32(0.9)), (5, np.float32(0.999))):
        p = float(beta) ** t.astype(np.float64)
        want = 1.0 / (1.0 - p)
        got = oracle.math(op, t).astype(np.float64)
        ulp_p = np.maximum(np.spacing(p.astype(np.float32)).astype(np.float64), 2.0 ** -25)   # 1 - p rounds at 2^-24 or finer
        bound = 2.5 * ulp_p / (1.0 - p) + 2e-7
        assert (np.abs(got / want - 1.0) <= bound).all(), (op, float(np.abs(got / want - 1.0).max()))
    # t = 1: the power is the float constant itself and 1 - beta is exact (the reference's value)
    assert oracle.math(4, np.array([1], np.float32))[0] == np.float32(1.0) / (np.float32(1.0) - np.float32(0.9))
    assert oracle.math(5, np.array([1], np.float32))[0] == np.float32(1.0) / (np.float32(1.0) - np.float32(0.999))
    wrong = 1.0 / (1.0 - 0.999 ** 2.0)    # the double-constant form misses by > 5e-6 at t = 2
    assert abs(oracle.math(5, np.array([2], np.float32))[0] / wrong - 1.0) > 5e-6
