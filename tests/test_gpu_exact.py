"""The exact method (method 0; src/core/continuous_tree_grower.cu, src/io/io.cu:437-482 of the
reference): every distinct value of a feature is a candidate threshold.  The reference's exact
goldens, and seeded data against the CPU checker's exact mode, bit for bit."""
import numpy as np
import pytest

from conftest import load_golden
from test_gpu_parity import _golden_cases, arb  # noqa: F401

pytestmark = pytest.mark.gpu


def test_golden_exact_regression(arb):
    fx = load_golden("exact_regression_boston10.json")     # tests/py/test_regression.py
    _golden_cases(arb, fx, np.array(fx["X"], np.float32), np.array(fx["y"], np.float32))


def test_golden_exact_logistic(arb):
    fx = load_golden("exact_logistic_iris.json")           # tests/py/test_logresression.py
    _golden_cases(arb, fx, np.array(fx["X"], np.float32), (np.array(fx["target"]) != 2).astype(np.float32))


@pytest.mark.parametrize("double_precision", [True, False])
@pytest.mark.parametrize("hist_size", [255, 1023])
def test_sklearn_goldens_with_the_exact_method(arb, double_precision, hist_size):
    # tests/py/test_sklearn_classification.py:9-61 and test_sklearn_regressor.py:9-40, method='exact'
    fx = load_golden("sklearn_classification_iris.json")
    X, y = np.array(fx["X"], np.float32), np.array(fx["target"]) != 2
    params = {k: v for k, v in fx["params"].items() if not (isinstance(v, str) and v.startswith("$"))}
    m = arb.ArboretumClassifier(double_precision=double_precision, method="exact", hist_size=hist_size, **params)
    data = arb.DMatrix(X, y=y)
    m.fit(data, y)
    assert np.allclose(m.predict(data), fx["y_pred"])
    fr = load_golden("hist_regression_boston10.json")
    X, y = np.array(fr["X"], np.float32), np.array(fr["y"], np.float32)
    r = arb.ArboretumRegression(max_depth=1, learning_rate=0.99999, n_estimators=1, verbosity=0,
                                min_child_weight=1.0, min_leaf_size=1, colsample_bytree=1.0, l1=0, l2=0,
                                double_precision=double_precision, method='exact', hist_size=hist_size)
    r.fit(arb.DMatrix(X, y=y), y)
    assert np.allclose(r.predict(arb.DMatrix(X)), fr["cases"]["test_single_tree_depth_1"]["true_values"][0])


def _data(n, F, distinct, objective, seed):
    rng = np.random.default_rng(seed)
    X = rng.integers(0, distinct, size=(n, F)).astype(np.float32) * 0.37 - 11.0   # `distinct` values per column
    X[:, 0] = rng.integers(0, 3, size=n)                                           # a column with three
    s = X[:, 1] * 0.1 + np.sin(X[:, 2]) + X[:, 0]
    y = (s + 0.3 * rng.normal(size=n)).astype(np.float32) if objective == 0 else \
        (rng.random(n) < 1 / (1 + np.exp(-(s - s.mean())))).astype(np.float32)
    return X, y


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("n,F,distinct,depth", [(5000, 6, 200, 5), (20000, 5, 256, 6), (30000, 4, 1500, 5),
                                                (40000, 3, 4096, 4), (257, 9, 257, 3)])
def test_exact_matches_the_checker(arb, oracle, objective, n, F, distinct, depth):
    # up to 256 distinct values per feature the ranks take 8 bits (fused kernels), beyond that
    # 16 bits (up to 4096 histogram slots per feature)
    X, y = _data(n, F, distinct, objective, seed=n + distinct)
    cfg = {"objective": objective, "method": 0, "internals": {"double_precision": True, "hist_size": 16},
           "tree": {"max_depth": depth, "eta": 0.4, "lambda": 1.0, "min_child_weight": 1.0}}
    ob = oracle.Booster(X, y=y, config=cfg)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    for r in range(3):
        ob.grow(1)
        g.grow_tree()
        to, tg = ob.tree(r), g.tree(r)
        for key in ("fid", "quantized", "threshold", "gain"):
            assert np.array_equal(to[key], tg[key]), (key, r)
        assert np.array_equal(to["weights"], tg["weights"], equal_nan=True)
        assert np.array_equal(ob.leaf(), g.leaves())
        assert np.array_equal(ob.yhat(), g.train_yhat())
    # thresholds are values of the data: the smallest value that goes right
    used = tg["quantized"] >= 0
    for f, thr in zip(tg["fid"][used], tg["threshold"][used]):
        assert thr in X[:, f]
    assert np.allclose(ob.predict(X), g.predict(data), atol=1e-6)
    # prediction on the training rows reproduces the tracked y_hat: value < threshold goes left
    raw = g.train_yhat()
    want = raw if objective == 0 else 1 / (1 + np.exp(-raw.astype(np.float64)))
    assert np.allclose(g.predict(data), want, atol=1e-6)


def test_exact_limits_are_errors(arb):
    rng = np.random.default_rng(0)
    X = rng.normal(size=(6000, 2)).astype(np.float32)          # 6000 distinct values per column
    y = X[:, 0].copy()
    g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}}, arb.DMatrix(X, y=y))
    with pytest.raises(arb.ArboretumError, match="up to 4096 distinct values"):
        g.grow_tree()
    X = np.round(X, 1)
    X[5, 1] = np.nan
    g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}}, arb.DMatrix(X, y=y))
    with pytest.raises(arb.ArboretumError, match="missing values"):
        g.grow_tree()
    bins = rng.integers(0, 9, size=(100, 3), dtype=np.uint8)
    g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}},
                   arb.DMatrix(bins, y=np.arange(100, dtype=np.float32), quantized=True))
    with pytest.raises(arb.ArboretumError, match="float features"):
        g.grow_tree()
