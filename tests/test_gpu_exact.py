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


def _continuous(n, F, objective, seed):
    """Columns of n draws from a continuous law: (almost) every value of a column is distinct."""
    rng = np.random.default_rng(seed)
    X = rng.normal(size=(n, F)).astype(np.float32)
    X[:, F - 1] = rng.integers(0, 5, size=n)           # and one column of five values
    s = X[:, 0] + np.sin(3 * X[:, 1]) + 0.5 * X[:, F - 1]
    y = (s + 0.3 * rng.normal(size=n)).astype(np.float32) if objective == 0 else \
        (rng.random(n) < 1 / (1 + np.exp(-s))).astype(np.float32)
    return X, y


def _same_trees(ob, g, rounds, data=None):
    for r in range(rounds):
        ob.grow(1)
        g.grow_tree()
        to, tg = ob.tree(r), g.tree(r)
        for key in ("fid", "quantized", "threshold", "gain"):
            assert np.array_equal(to[key], tg[key]), (key, r)
        assert np.array_equal(to["weights"], tg["weights"], equal_nan=True)
        assert np.array_equal(ob.leaf(), g.leaves())
        assert np.array_equal(ob.yhat(), g.train_yhat())


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("double_precision", [True, False])
@pytest.mark.parametrize("n,F,depth", [(30000, 4, 5), (60000, 3, 7), (5000, 5, 2)])
def test_sorted_lists_match_the_checker(arb, oracle, objective, double_precision, n, F, depth):
    # more than 4096 distinct values per feature (5000 rows: forced): every feature keeps its rows
    # sorted by value instead of a histogram over ranks
    X, y = _continuous(n, F, objective, seed=n + depth)
    assert len(np.unique(X[:, 0])) > min(n, 4096) * 0.99
    cfg = {"objective": objective, "method": 0,
           "internals": {"double_precision": double_precision, "exact_sort": 1 if n <= 5000 else -1},
           "tree": {"max_depth": depth, "eta": 0.4, "lambda": 1.0, "min_child_weight": 1.0, "min_leaf_size": 3}}
    ob = oracle.Booster(X, y=y, config=cfg)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    _same_trees(ob, g, 3)
    tg = g.tree(2)
    used = tg["quantized"] >= 0
    assert used.sum() >= (2 ** depth - 1) * 3 // 4       # (most nodes are split: the trees are not trivial)
    for f, thr in zip(tg["fid"][used], tg["threshold"][used]):
        assert thr in X[:, f]                          # the smallest value that goes right
    assert np.allclose(ob.predict(X), g.predict(data), atol=1e-6)
    raw = g.train_yhat()
    want = raw if objective == 0 else 1 / (1 + np.exp(-raw.astype(np.float64)))
    assert np.allclose(g.predict(data), want, atol=1e-6)


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("n,F,distinct,depth", [(20000, 5, 256, 6), (30000, 4, 1500, 5), (257, 9, 257, 3), (70, 3, 9, 4)])
def test_sorted_lists_and_rank_histograms_grow_the_same_trees(arb, oracle, objective, n, F, distinct, depth):
    # where both paths can run (up to 4096 distinct values) they agree with each other and the checker
    X, y = _data(n, F, distinct, objective, seed=7 * n + distinct)
    trees = []
    for by_sorting in (1, 0):
        cfg = {"objective": objective, "method": 0, "internals": {"double_precision": True, "exact_sort": by_sorting},
               "tree": {"max_depth": depth, "eta": 0.4, "lambda": 0.5, "min_child_weight": 0.5, "gamma_absolute": 0.01}}
        g = arb.Garden(cfg, arb.DMatrix(X, y=y))
        _same_trees(oracle.Booster(X, y=y, config=cfg), g, 2)
        trees.append(g.tree(1))
    for key in trees[0]:
        assert np.array_equal(trees[0][key], trees[1][key], equal_nan=True), key


def test_sorted_lists_with_column_sampling_and_soft_max(arb, oracle):
    rng = np.random.default_rng(11)
    X = rng.normal(size=(12000, 6)).astype(np.float32)
    labels = ((X[:, 0] > 0).astype(np.int64) + (X[:, 2] > 0.5) + (X[:, 4] < -0.3)).astype(np.uint8)
    cfg = {"objective": 3, "method": 0, "internals": {"double_precision": True, "seed": 5},
           "tree": {"max_depth": 4, "eta": 0.5, "labels_count": 4, "colsample_bytree": 0.7, "colsample_bylevel": 0.7}}
    ob = oracle.Booster(X, labels=labels, config=cfg)
    g = arb.Garden(cfg, arb.DMatrix(X, labels=labels))
    for r in range(2):
        ob.grow(1)
        g.grow_tree()
        for t in range(4 * r, 4 * r + 4):
            to, tg = ob.tree(t), g.tree(t)
            for key in ("fid", "quantized", "threshold", "gain"):
                assert np.array_equal(to[key], tg[key]), (key, t)
            assert np.array_equal(to["weights"], tg["weights"], equal_nan=True)
        assert np.array_equal(ob.yhat(), g.train_yhat())


@pytest.mark.parametrize("seed", range(16))
def test_sorted_lists_on_random_configurations(arb, oracle, seed):
    # columns of every kind (continuous, rounded so that values repeat, a handful of values, one
    # constant), every tree parameter drawn at random: ties, empty and tiny nodes, rejected splits
    rng = np.random.default_rng(1000 + seed)
    n, F = int(rng.integers(40, 30000)), int(rng.integers(1, 9))
    X = np.empty((n, F), np.float32)
    for f in range(F):
        kind = rng.integers(0, 4) if f else 0
        col = rng.normal(size=n) * 10 ** rng.uniform(-3, 3)
        X[:, f] = col if kind == 0 else np.round(col, 0) if kind == 1 else rng.integers(0, 4, size=n) if kind == 2 else 1.5
    objective = int(rng.integers(0, 2))
    s = X[:, 0] / np.abs(X[:, 0]).max() * 3 + (X[:, F - 1] > np.median(X[:, F - 1]))
    y = (s + 0.3 * rng.normal(size=n)).astype(np.float32) if objective == 0 else \
        (rng.random(n) < 1 / (1 + np.exp(-s))).astype(np.float32)
    cfg = {"objective": objective, "method": 0,
           "internals": {"double_precision": bool(rng.integers(0, 2)), "exact_sort": 1, "seed": int(rng.integers(0, 99))},
           "tree": {"max_depth": int(rng.integers(1, 8)), "eta": float(rng.uniform(0.05, 1.0)),
                    "lambda": float(rng.choice([0.0, 0.5, 2.0])), "alpha": float(rng.choice([0.0, 0.0, 0.3])),
                    "min_child_weight": float(rng.choice([0.0, 1.0, 5.0])), "min_leaf_size": int(rng.choice([0, 1, 2, 20])),
                    "gamma_absolute": float(rng.choice([0.0, 0.0, 0.5])), "gamma_relative": float(rng.choice([0.0, 0.0, 0.01])),
                    "max_leaf_weight": float(rng.choice([0.0, 0.0, 0.7])),
                    "colsample_bytree": float(rng.choice([1.0, 1.0, 0.8])) if F > 2 else 1.0,
                    "colsample_bylevel": float(rng.choice([1.0, 1.0, 0.8])) if F > 2 else 1.0}}
    _same_trees(oracle.Booster(X, y=y, config=cfg), arb.Garden(cfg, arb.DMatrix(X, y=y)), 3)


@pytest.mark.parametrize("objective", [0, 1])
def test_sorted_lists_over_many_work_items(arb, oracle, objective):
    # a million rows: several hundred work items per list at the root (the sums and left counts of a
    # node's items are scanned in rounds of 64), many rows per distinct value, nodes of every size
    n = 1_000_000
    rng = np.random.default_rng(21 + objective)
    X = np.empty((n, 3), np.float32)
    X[:, 0] = np.round(rng.normal(size=n) * 9000.0)            # about 50 000 distinct values
    X[:, 1] = np.round(rng.exponential(size=n) * 3000.0)       # skewed: many rows share the small values
    X[:, 2] = rng.integers(0, 7, size=n)
    s = np.tanh(X[:, 0] / 9000.0) + (X[:, 1] > 2000.0) + 0.2 * X[:, 2]
    y = (s + 0.3 * rng.normal(size=n)).astype(np.float32) if objective == 0 else \
        (rng.random(n) < 1 / (1 + np.exp(-(s - 1.0)))).astype(np.float32)
    cfg = {"objective": objective, "method": 0, "internals": {"double_precision": True},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0, "min_child_weight": 1.0}}
    ob = oracle.Booster(X, y=y, config=cfg)
    assert 4096 < ob.params.hist_size < 65536
    _same_trees(ob, arb.Garden(cfg, arb.DMatrix(X, y=y)), 2)


@pytest.mark.parametrize("objective", [0, 1])
def test_sorted_lists_match_the_checker_beyond_16_bit_ranks(arb, oracle, objective):
    # 100 000 distinct values per feature: the checker's exact mode with 32-bit ranks
    n = 100000
    rng = np.random.default_rng(5 + objective)
    X = (rng.permutation(2 * n).reshape(n, 2) / 8.0).astype(np.float32)        # all distinct, exact in float32
    s = np.sin(X[:, 0] / 3000.0) + (X[:, 1] > 9000.0)
    y = (s + 0.2 * rng.normal(size=n)).astype(np.float32) if objective == 0 else \
        (rng.random(n) < 1 / (1 + np.exp(-2 * s + 1))).astype(np.float32)
    cfg = {"objective": objective, "method": 0, "internals": {"double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.5, "lambda": 1.0, "min_child_weight": 1.0}}
    ob = oracle.Booster(X, y=y, config=cfg)
    assert ob.params.hist_size == n
    _same_trees(ob, arb.Garden(cfg, arb.DMatrix(X, y=y)), 2)


def test_sorted_lists_beyond_the_checker(arb):
    # 300 000 distinct values per feature and six levels, more than the checker's rank histograms
    # hold in reasonable memory: what does not depend on the size.  A strictly increasing map of a feature changes no rank, so the trees
    # keep their features, ranks, gains, weights and leaves, and every threshold maps with it; the
    # root split is the best of all places by a float64 restatement of the squared-error gain;
    # prediction from the thresholds reproduces the tracked y_hat (rank <= q <=> value < threshold).
    n = 300000
    rng = np.random.default_rng(3)
    X = rng.permutation(n * 3).reshape(n, 3).astype(np.float32) / 4.0      # distinct, exact in float32
    y = (np.sin(X[:, 0] / 40000.0) + (X[:, 1] > 120000.0) + 0.1 * rng.normal(size=n)).astype(np.float32)
    Z = X.copy()
    Z[:, 0] = X[:, 0] * 2.0 - 1000.0
    Z[:, 1] = np.sqrt(X[:, 1].astype(np.float64) + 1.0).astype(np.float32) * 64.0
    assert all(len(np.unique(Z[:, f])) == n for f in range(3))
    cfg = {"objective": 0, "method": 0, "internals": {"double_precision": True},
           "tree": {"max_depth": 6, "eta": 0.5, "lambda": 0.0, "min_child_weight": 0.0, "min_leaf_size": 1,
                    "initial_y": 0.0}}
    grown = []
    for M in (X, Z):
        data = arb.DMatrix(M, y=y)
        g = arb.Garden(cfg, data)
        for _ in range(2):
            g.grow_tree()
        assert np.allclose(g.predict(data), g.train_yhat(), atol=1e-5)
        grown.append((g.tree(0), g.tree(1), g.leaves(), g.train_yhat()))
    for a, b in zip(grown[0][:2], grown[1][:2]):
        for key in ("fid", "quantized", "gain", "weights"):
            assert np.array_equal(a[key], b[key], equal_nan=True), key
    assert np.array_equal(grown[0][2], grown[1][2]) and np.array_equal(grown[0][3], grown[1][3])
    t0 = grown[0][0]
    # the root by brute force: gain = GL^2 / HL + GR^2 / HR - GT^2 / HT with H = count (lambda 0).
    # The builder rounds each of the three terms to float, so its choice may be any place whose
    # gain is within that rounding of the best one.
    best, chosen = -1.0, None
    GT = float(y.astype(np.float64).sum())
    for f in range(3):
        order = np.argsort(X[:, f], kind="stable")
        GL = np.cumsum(y[order].astype(np.float64))[:-1]
        cl = np.arange(1, n, dtype=np.float64)
        gain = GL ** 2 / cl + (GT - GL) ** 2 / (n - cl) - GT ** 2 / n
        best = max(best, float(gain.max()))
        if f == int(t0["fid"][0]):
            k = int(np.searchsorted(X[order, f], t0["threshold"][0]))      # the first row that goes right
            assert X[order[k], f] == t0["threshold"][0] and int(t0["quantized"][0]) == k - 1
            chosen = float(gain[k - 1])
    assert chosen is not None and chosen >= best * (1 - 1e-6)
    assert np.isclose(t0["gain"][0], best, rtol=1e-5)


def test_exact_limits_are_errors(arb):
    rng = np.random.default_rng(0)
    X = rng.normal(size=(6000, 2)).astype(np.float32)          # 6000 distinct values per column
    y = X[:, 0].copy()
    g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}, "internals": {"exact_sort": 0}},
                   arb.DMatrix(X, y=y))
    with pytest.raises(arb.ArboretumError, match="up to 4096 distinct values"):
        g.grow_tree()
    data = arb.DMatrix(X, y=y)
    g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}}, data)
    g.grow_tree()                                               # sorted row lists: no bin ids to show
    with pytest.raises(arb.ArboretumError, match="no bin ids"):
        data.bins()
    g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}, "internals": {"upload_features": False}},
                   arb.DMatrix(X, y=y))
    with pytest.raises(arb.ArboretumError, match="not built for streamed"):
        g.grow_tree()
    X = np.round(X, 1)
    X[5, 1] = np.nan
    for by_sorting in (-1, 1):
        g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}, "internals": {"exact_sort": by_sorting}},
                       arb.DMatrix(X, y=y))
        with pytest.raises(arb.ArboretumError, match="missing values"):
            g.grow_tree()
    bins = rng.integers(0, 9, size=(100, 3), dtype=np.uint8)
    g = arb.Garden({"objective": 0, "method": 0, "tree": {"max_depth": 2}},
                   arb.DMatrix(bins, y=np.arange(100, dtype=np.float32), quantized=True))
    with pytest.raises(arb.ArboretumError, match="float features"):
        g.grow_tree()
