"""The five benchmark configurations at sizes the oracle finishes in seconds:
same generators, objectives and tree parameters, fewer rows and trees.  The
HIP path must reproduce the oracle bit for bit on each of them."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

from test_gpu_parity import assert_same_training  # noqa: E402

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


def test_config_0_regression_plumbing(arb, oracle):
    # exactly as specified: 10,000 x 28 ~ N(0,1), y = X.w + 0.1 N(0,1), squared error, 256 bins,
    # max_depth 6, eta 0.3, lambda 1, 10 trees
    rng = np.random.default_rng(0)
    X = rng.standard_normal(size=(10000, 28), dtype=np.float32)
    w = rng.standard_normal(28)
    y = (X @ w + 0.1 * rng.standard_normal(10000)).astype(np.float32)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 256, "double_precision": True},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=10)
    # the trees learn: the training error falls well below the variance of y
    pred = g.predict(g.data)
    assert np.mean((pred - y) ** 2) < 0.25 * np.var(y)


def test_config_1_binary_classification(arb, oracle):
    import bench
    X, y = bench.make_workload(300000, 28)
    assert 0.45 < y.mean() < 0.6
    assert_same_training(arb, oracle, X, y, bench.config(8, 256), rounds=4, check_hist=False)


def test_config_2_missing_values_and_categories(arb, oracle):
    # 200 features, 30 % NaN, half Uniform(0,1), half Zipf(1.1) categories 0..49; piecewise-constant
    # regression target; 64 bins (+ the missing bin), max_depth 10.  Missing values go right, as in
    # the reference (no learned default direction).
    rng = np.random.default_rng(2)
    n, F = 60000, 200
    X = rng.random(size=(n, F), dtype=np.float32)
    cats = np.minimum(rng.zipf(1.1, size=(n, F // 2)) - 1, 49).astype(np.float32)
    X[:, F // 2:] = cats
    y = np.zeros(n, dtype=np.float32)
    for _ in range(20):
        f = int(rng.integers(0, F))
        t = float(rng.choice(X[:1000, f]))
        y += np.where(X[:, f] > t, rng.normal(), rng.normal()).astype(np.float32)
    y += 0.1 * rng.standard_normal(n).astype(np.float32)
    X[rng.random(size=(n, F)) < 0.3] = np.nan
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 64, "double_precision": True},
           "tree": {"max_depth": 10, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2, check_hist=False)


def test_config_3_multiclass_softmax(arb, oracle):
    rng = np.random.default_rng(3)
    n, F, K = 30000, 100, 10
    X = rng.standard_normal(size=(n, F), dtype=np.float32)
    W = rng.standard_normal(size=(F, K))
    labels = np.argmax(X @ W + rng.gumbel(size=(n, K)), axis=1).astype(np.uint8)
    cfg = {"objective": 4, "method": 1, "internals": {"hist_size": 256, "double_precision": True},
           "tree": {"max_depth": 6, "eta": 0.2, "lambda": 1.0, "labels_count": K}}
    ob = oracle.Booster(X, labels=labels, config=cfg)
    data = arb.DMatrix(X, labels=labels)
    g = arb.Garden(cfg, data)
    for r in range(2):
        ob.grow(1)
        g.grow_tree()
    for t in range(2 * K):
        to, tg = ob.tree(t), g.tree(t)
        for key in ("fid", "quantized", "threshold", "gain", "weights"):
            assert np.array_equal(to[key], tg[key], equal_nan=True), (key, t)
    assert np.array_equal(ob.yhat(), g.train_yhat())
    assert np.allclose(ob.predict(X), g.predict(data), atol=1e-6)


def test_config_4_out_of_core_prequantised(arb, oracle):
    # 128 pre-quantised uint8 columns, uniform or Binomial(255, 0.3); labels from a random depth-6
    # tree with 10 % flips; bins streamed from pinned host blocks; max_depth 8
    import bench
    bins, y = bench.make_stream_workload(200000, 128)
    cfg = bench.config(8, 256)
    cfg["internals"]["upload_features"] = False
    cfg["internals"]["stream_block_rows"] = 65536
    ob = oracle.Booster(bins, y=y, config=cfg, binned=True)
    data = arb.DMatrix(bins, y=y, quantized=True)
    g = arb.Garden(cfg, data)
    for r in range(3):
        ob.grow(1)
        g.grow_tree()
        to, tg = ob.tree(r), g.tree(r)
        for key in ("fid", "quantized", "gain", "weights"):
            assert np.array_equal(to[key], tg[key], equal_nan=True), (key, r)
        assert np.array_equal(ob.leaf(), g.leaves())
        assert np.array_equal(ob.yhat(), g.train_yhat())
