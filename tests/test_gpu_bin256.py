"""hist_size 256 on a feature that fills all 256 value bins AND has missing values: 257 bin ids
(NaN -> bin `size`, src/core/cuda_helpers.h:207-222; the reference switches to 16-bit ids at this
hist_size, src/core/garden.cu:514-523).  The HIP path keeps 8-bit ids plus a ninth bit per feature
and must equal the CPU checker bit for bit on every path that reads a row: fused levels, the last level, the last pass with and without the next root histogram,
un-fused levels (no sibling subtraction), streamed blocks.  Needs an MI355X: run with `-m gpu`."""
import numpy as np
import pytest

from test_gpu_parity import arb, assert_same_training  # noqa: F401  (fixture)

pytestmark = pytest.mark.gpu


def _data(n, F, objective, seed, nan_rows=40, informative_nan=True):
    """Continuous columns with a handful of missing values each, few enough that every column still
    fills its 256 value bins (fewer than n / 256 of them).  With informative_nan the rows missing in
    feature 1 carry nearly all the signal, so 'missing against the rest' (bin 255 of that feature)
    is the best split of the root."""
    rng = np.random.default_rng(seed)
    X = rng.normal(size=(n, F)).astype(np.float32)
    s = 0.05 * X[:, 0] + 0.05 * X[:, F - 1] * X[:, F // 2]
    miss1 = None
    for f in range(F):
        idx = rng.choice(n, size=nan_rows, replace=False)
        X[idx, f] = np.nan
        if f == min(1, F - 1):
            miss1 = idx
    s = np.nan_to_num(s)
    if informative_nan and nan_rows:
        s[miss1] += 8.0
    if objective == 0:
        y = (s + 0.2 * rng.normal(size=n)).astype(np.float32)
    else:
        y = (rng.random(n) < 1 / (1 + np.exp(-(s - 2.0)))).astype(np.float32)
    return X, y


def _cfg(objective, depth, trick=True, upload=True, dp=True, **internals):
    return {"objective": objective, "method": 1,
            "internals": dict({"hist_size": 256, "double_precision": dp, "use_hist_subtraction_trick": trick,
                               "upload_features": upload}, **internals),
            "tree": {"max_depth": depth, "eta": 0.3, "lambda": 1.0, "min_child_weight": 0.0}}


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("F", [1, 5, 28, 32])
def test_ninth_bit_ids_resident(arb, oracle, objective, F):
    X, y = _data(40000, F, objective, seed=F)
    ob, g = assert_same_training(arb, oracle, X, y, _cfg(objective, 5), rounds=3)
    assert g.data.bin_layout() == (8, 257)
    assert ob.bins().max() == 256
    assert g.tree(0)["quantized"][0] == 255     # 'missing against the rest' of feature min(1, F - 1)


@pytest.mark.parametrize("objective", [0, 1])
def test_ninth_bit_ids_without_inspection(arb, oracle, objective):
    # inspection off: the last pass also builds the next root histogram (logistic), gradients stay packed
    X, y = _data(60000, 28, objective, seed=11)
    ob, g = assert_same_training(arb, oracle, X, y, _cfg(objective, 6, dp=False), rounds=5, check_hist=False)
    assert g.data.bin_layout() == (8, 257)
    assert g.tree(0)["quantized"][0] == 255


def test_ninth_bit_ids_labels_outside_0_1_keep_two_gradient_arrays(arb, oracle):
    X, y = _data(30000, 9, 1, seed=3)
    y = y * 1.5 - 0.25
    assert_same_training(arb, oracle, X, y, _cfg(1, 5), rounds=3, check_hist=False)


@pytest.mark.parametrize("objective", [0, 1])
def test_ninth_bit_ids_without_sibling_subtraction(arb, oracle, objective):
    X, y = _data(30000, 13, objective, seed=5)
    assert_same_training(arb, oracle, X, y, _cfg(objective, 4, trick=False), rounds=2)


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("block_rows", [4096, 1 << 20])
def test_ninth_bit_ids_streamed(arb, oracle, objective, block_rows):
    X, y = _data(30000, 12, objective, seed=7)
    ob, g = assert_same_training(arb, oracle, X, y, _cfg(objective, 4, upload=False, stream_block_rows=block_rows),
                                 rounds=2)
    assert g.data.bin_layout() == (8, 257)


def test_ninth_bit_ids_softmax(arb, oracle):
    rng = np.random.default_rng(2)
    n, F, K = 20000, 6, 3
    X = rng.normal(size=(n, F)).astype(np.float32)
    labels = np.argmax(X[:, :K] + rng.gumbel(size=(n, K)), axis=1).astype(np.uint8)
    X[rng.choice(n, size=25, replace=False), 2] = np.nan
    cfg = _cfg(4, 4)
    cfg["tree"]["labels_count"] = K
    ob = oracle.Booster(X, labels=labels, config=cfg)
    data = arb.DMatrix(X, labels=labels)
    g = arb.Garden(cfg, data)
    for r in range(2):
        ob.grow(1)
        g.grow_tree()
    assert data.bin_layout() == (8, 257)
    for t in range(2 * K):
        a, b = ob.tree(t), g.tree(t)
        for k in ("fid", "quantized", "threshold", "gain", "weights"):
            assert np.array_equal(a[k], b[k]), (t, k)
    assert np.array_equal(ob.yhat(), g.train_yhat())


def test_one_missing_value_keeps_the_headline_kernels(arb, oracle):
    # a single NaN in one of 28 continuous features: still 8-bit ids (with the ninth bit), same trees
    # as the checker; the same for a matrix wider than 32 features
    X, y = _data(50000, 28, 1, seed=21, nan_rows=0, informative_nan=False)
    X[123, 4] = np.nan
    ob, g = assert_same_training(arb, oracle, X, y, _cfg(1, 6), rounds=2, check_hist=False)
    assert g.data.bin_layout() == (8, 257)
    Xw = np.random.default_rng(1).normal(size=(20000, 40)).astype(np.float32)
    Xw[5, 7] = np.nan
    yw = (Xw[:, 0] > 0).astype(np.float32)
    ob, g = assert_same_training(arb, oracle, Xw, yw, _cfg(1, 3), rounds=1, check_hist=False)
    assert g.data.bin_layout() == (8, 257)


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("F,depth", [(33, 5), (40, 1), (64, 4), (100, 5), (130, 3)])
def test_ninth_bit_ids_wide_matrices(arb, oracle, objective, F, depth):
    # more than 32 features: a ninth-bit word per 32 features, rows in place as records (the words
    # ride in the record), ids of 256 left out of the histograms (no candidate's left side holds
    # them) and reported from the node totals; max_depth 1 takes the column kernels alone
    X, y = _data(30000, F, objective, seed=100 + F)
    ob, g = assert_same_training(arb, oracle, X, y, _cfg(objective, depth), rounds=2)
    assert g.data.bin_layout() == (8, 257)
    assert ob.bins().max() == 256
    assert g.tree(0)["quantized"][0] == 255
    assert_same_training(arb, oracle, X, y, _cfg(objective, depth, trick=False), rounds=2, check_hist=False)


@pytest.mark.parametrize("resident", [0, -1])
def test_ninth_bit_ids_wide_matrices_streamed(arb, oracle, resident):
    X, y = _data(30000, 70, 1, seed=170)
    cfg = _cfg(1, 4, upload=False, stream_block_rows=8192, stream_resident_bytes=resident)
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=2)
    assert g.data.bin_layout() == (8, 257)
    assert g.tree(0)["quantized"][0] == 255


def test_ninth_bit_ids_wide_softmax(arb, oracle):
    rng = np.random.default_rng(12)
    n, F, K = 20000, 48, 3
    X = rng.normal(size=(n, F)).astype(np.float32)
    labels = np.argmax(X[:, :K] + rng.gumbel(size=(n, K)), axis=1).astype(np.uint8)
    X[rng.choice(n, size=25, replace=False), 40] = np.nan
    cfg = _cfg(4, 4)
    cfg["tree"]["labels_count"] = K
    ob = oracle.Booster(X, labels=labels, config=cfg)
    data = arb.DMatrix(X, labels=labels)
    g = arb.Garden(cfg, data)
    for r in range(2):
        ob.grow(1)
        g.grow_tree()
    assert data.bin_layout() == (8, 257)
    for t in range(2 * K):
        a, b = ob.tree(t), g.tree(t)
        for k in ("fid", "quantized", "threshold", "gain", "weights"):
            assert np.array_equal(a[k], b[k]), (t, k)
    assert np.array_equal(ob.yhat(), g.train_yhat())


def test_no_missing_values_no_ninth_bit(arb, oracle):
    X, y = _data(20000, 7, 1, seed=4, nan_rows=0, informative_nan=False)
    ob, g = assert_same_training(arb, oracle, X, y, _cfg(1, 4), rounds=1)
    assert g.data.bin_layout() == (8, 256)
