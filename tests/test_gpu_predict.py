"""Batch prediction on the GPU against the host walk (RegTree::Predict,
src/core/garden.h:70-90; Garden::Predict, src/core/garden.cu:643-657): the two
must agree bit for bit, and both with the CPU checker."""
import json

import numpy as np
import pytest

from test_gpu_parity import make_data

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


def both_ways(g, data, n_rounds=-1):
    g.predict_on_device(True)
    dev = g.predict(data, n_rounds)
    g.predict_on_device(False)
    host = g.predict(data, n_rounds)
    g.predict_on_device(True)
    assert dev.shape == host.shape
    assert np.array_equal(dev, host, equal_nan=True)
    return dev


@pytest.mark.parametrize("objective,nan_frac,n", [(0, 0.0, 5000), (1, 0.0, 70001), (1, 0.2, 1023), (0, 0.1, 1025)])
def test_device_walk_equals_host_walk_and_checker(arb, oracle, objective, nan_frac, n):
    X, y = make_data(n, 9, objective, seed=21 + n, nan_frac=nan_frac)
    cfg = {"objective": objective, "method": 1, "internals": {"hist_size": 64, "double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0, "min_child_weight": 0.0}}
    ob = oracle.Booster(X, y=y, config=cfg)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    for _ in range(6):
        ob.grow(1)
        g.grow_tree()
    # new rows, with values the training matrix never held
    Xn, _ = make_data(3 * n // 2 + 7, 9, objective, seed=5, nan_frac=nan_frac)
    Xn[::17, 3] = np.inf
    Xn[::19, 4] = -np.inf
    new = arb.DMatrix(Xn)
    for rounds in (-1, 1, 4, 100):
        p = both_ways(g, new, rounds)
        assert np.allclose(p, ob.predict(Xn, rounds if rounds > 0 else -1), rtol=0, atol=1e-6, equal_nan=True)
    both_ways(g, data)


def test_softmax_rows_by_labels(arb):
    rng = np.random.default_rng(4)
    n, F, K = 20000, 12, 5
    X = rng.standard_normal(size=(n, F), dtype=np.float32)
    labels = np.argmax(X[:, :K] + 0.5 * rng.gumbel(size=(n, K)), axis=1).astype(np.uint8)
    cfg = {"objective": 4, "method": 1, "internals": {"hist_size": 64, "double_precision": True},
           "tree": {"max_depth": 4, "eta": 0.3, "lambda": 1.0, "labels_count": K}}
    data = arb.DMatrix(X, labels=labels)
    g = arb.Garden(cfg, data)
    for _ in range(3):
        g.grow_tree()
    p = both_ways(g, data)
    assert p.shape == (n, K) and np.allclose(p.sum(axis=1), 1.0, atol=1e-5)
    # n_rounds counts trees, not rounds (garden.cu:646-650): a partial round is allowed
    both_ways(g, data, 7)
    assert (np.argmax(p, axis=1) == labels).mean() > 0.6


def test_several_row_blocks(arb):
    # 28 features: blocks of 299,008 rows, so 700,001 rows take three blocks, the last one ragged
    import bench
    X, y = bench.make_workload(700001, 28)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(bench.config(8, 256), data)
    for _ in range(25):   # more trees than one LDS chunk holds at this depth
        g.grow_tree()
    p = both_ways(g, data)
    dev = 1.0 / (1.0 + np.exp(-g.train_yhat().astype(np.float64)))
    # training walks the bins (x <= threshold goes left), prediction the floats (x < threshold, as the
    # reference): a value equal to a threshold, which a midpoint of two neighbouring floats can be,
    # takes the other side, so a few rows in a million may differ
    assert (np.abs(p - dev) > 1e-6).mean() < 1e-4


def test_repeated_prediction_on_the_same_matrix(arb):
    # the columns of the last matrix stay on the device: a second call on it (with more trees, as
    # an evaluation loop does), a call on another matrix, and the first one again
    Xa, ya = make_data(50000, 7, 1, seed=3, nan_frac=0.05)
    Xb, _ = make_data(1300, 7, 1, seed=4)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 32, "double_precision": True},
           "tree": {"max_depth": 4, "eta": 0.3, "lambda": 1.0}}
    train = arb.DMatrix(Xa, y=ya)
    a, b = arb.DMatrix(Xa), arb.DMatrix(Xb)
    g = arb.Garden(cfg, train)
    seen = []
    for r in range(3):
        g.grow_tree()
        seen.append(both_ways(g, a))
        if r == 1:
            both_ways(g, b)
    assert not np.array_equal(seen[0], seen[1]) and not np.array_equal(seen[1], seen[2])
    both_ways(g, a, 1)
    del a
    c = arb.DMatrix(Xb[:700] * 2)      # possibly at the address of the matrix just freed
    both_ways(g, c)


def _random_model(rng, depths, F, fid_max):
    model = []
    for d in depths:           # d = internal depth: 2^(d-1) - 1 split nodes
        internal = (1 << (d - 1)) - 1
        nodes = []
        for i in range(internal):
            thr = float(np.float32(rng.normal()))
            node = {"id": i, "leaf": False, "left": 2 * i + 1, "right": 2 * i + 2,
                    "threshold": None if rng.random() < 0.05 else thr, "fid": int(rng.integers(0, fid_max))}
            nodes.append(node)
        for i in range(internal + 1):
            nodes.append({"id": internal + i, "leaf": True, "idx": i})
        weights = [float(np.float32(w)) for w in rng.normal(size=internal + 1)]
        model.append({"nodes": nodes, "weights": weights, "depth": d})
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 16},
           "tree": {"max_depth": 3, "initial_y": 0.25}}
    return json.dumps({"configuration": cfg, "model": model})


def test_loaded_model_mixed_depths_foreign_features_and_trees_beyond_lds(arb):
    # depth 15 and 16: 16383 / 32767 nodes do not fit the LDS staging and are read from global memory,
    # between trees that do fit; feature ids 6 and 7 do not exist in the matrix and read as missing;
    # null thresholds load as +inf
    rng = np.random.default_rng(8)
    F = 6
    text = _random_model(rng, [3, 9, 15, 2, 16, 5, 5, 13, 14, 4], F, fid_max=F + 2)
    g = arb.load(text)
    X = rng.normal(size=(4099, F)).astype(np.float32)
    X[rng.random(X.shape) < 0.1] = np.nan
    data = arb.DMatrix(X)
    p = both_ways(g, data)
    assert np.isfinite(p).all() and np.unique(p).size > 1000
    both_ways(g, data, 3)
    both_ways(g, data, 5)


@pytest.mark.parametrize("upload", [True, False])
def test_prequantised_matrices(arb, upload):
    # bin ids are compared as floats against the thresholds, as the host walk does; the rows come from
    # the row-major bytes on the host or, once a streamed matrix has given them up, from its pinned blocks
    rng = np.random.default_rng(2)
    bins = rng.integers(0, 256, size=(70001, 9), dtype=np.uint8)
    y = ((bins[:, 0] > 100) ^ (bins[:, 5] > 30)).astype(np.float32)
    cfg = {"objective": 1, "method": 1,
           "internals": {"hist_size": 256, "double_precision": True, "upload_features": upload,
                         "stream_block_rows": 16384},
           "tree": {"max_depth": 4, "eta": 0.5, "lambda": 1.0}}
    data = arb.DMatrix(bins, y=y, quantized=True)
    fresh = arb.DMatrix(bins[::-1].copy(), quantized=True)   # never quantised: bytes on the host
    g = arb.Garden(cfg, data)
    for _ in range(5):
        g.grow_tree()
    p = both_ways(g, data)
    assert ((p > 0.5) == (y > 0.5)).mean() > 0.95
    assert np.array_equal(both_ways(g, fresh), p[::-1])
    both_ways(g, data, 2)
