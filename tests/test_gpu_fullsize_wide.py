"""BASELINE configs[2] (50 M x 200, 30 % missing, 65 bin ids, squared error, max_depth 10) and
configs[3] (20 M x 100, 10 soft-max classes, max_depth 6) at their full sizes, and the out-of-core
shape (64 M x 128 streamed).  The trees are checked through what holds at any size:
every row's leaf against a host walk of the tree over the bin ids, every leaf weight against its
definition on the rows the leaf holds, the prediction update against leaf weight + old value, and
the root split against histograms built with numpy (gain from the checker's pinned gain function,
ties as the reference breaks them); and the first trees of each against the CPU checker bit for bit."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


def _walk(tree, bins, depth):
    """Leaf of every row: bin > split bin goes right (child 2k+1 of the level), an unsplit node
    (bin -1) keeps everything left."""
    n = bins.shape[0]
    node = np.zeros(n, np.int64)
    rows = np.arange(n)
    for level in range(depth):
        at = (1 << level) - 1 + node
        fid, q = tree["fid"][at], tree["quantized"][at]
        right = (q >= 0) & (bins[rows, fid] > q)
        node = 2 * node + right
    return node.astype(np.uint32)


def _check_leaf_weights(tree, leaf, g, h, eta, lam):
    L = len(tree["weights"])
    G = np.bincount(leaf, weights=g.astype(np.float64), minlength=L)
    A = np.bincount(leaf, weights=np.abs(g).astype(np.float64), minlength=L)
    H = np.bincount(leaf, weights=h.astype(np.float64), minlength=L)
    held = np.bincount(leaf, minlength=L) > 0
    want = eta * G / (H + lam)
    tol = 1e-5 * eta * A / (H + lam) + 1e-7
    assert (np.abs(tree["weights"][held] - want[held]) <= tol[held]).all()
    return held.sum()


def _check_root_split(oracle, tree, bins, g, h, kind, features, slots, lam):
    """The root's (feature, bin, gain) against numpy histograms of the chosen feature and a few
    others: best gain per feature with ties to the highest bin, then the lowest feature."""
    n = bins.shape[0]
    g64, h64 = g.astype(np.float64), h.astype(np.float64)
    GT, HT = float(g64.sum()), float(h64.sum())
    f0, b0 = int(tree["fid"][0]), int(tree["quantized"][0])
    assert b0 >= 0
    best = {}
    for f in features:
        col = bins[:, f]
        hg = np.bincount(col, weights=g64, minlength=slots)
        hh = np.bincount(col, weights=h64, minlength=slots)
        hc = np.bincount(col, minlength=slots)
        pg, ph, pc = np.cumsum(hg), np.cumsum(hh), np.cumsum(hc)
        top, where = 0.0, -1
        for b in range(slots - 1):      # the last bin id holds the missing values and always goes right
            gain = oracle.lib().orc_gain(kind, float(pg[b]), float(ph[b]), int(pc[b]), GT, HT, n, 1, 1.0, 0.0, 0.0,
                                         lam, 0.0, 0.0)
            if gain > 0 and gain >= top:
                top, where = gain, b
        best[f] = (top, where)
    assert best[f0][1] == b0, "bin of the root split"
    assert tree["gain"][0] == pytest.approx(best[f0][0], rel=1e-4)
    for f, (gain, _) in best.items():
        if f != f0:
            assert gain < best[f0][0] * (1 + 1e-6) or (gain == pytest.approx(best[f0][0], rel=1e-6) and f > f0), \
                "feature %d beats the chosen feature %d" % (f, f0)


def _same_as_checker(ob, model, trees, leaves=True):
    """Every split, gain and leaf weight of the given trees, the leaf of every row and the
    predictions against the CPU checker, bit for bit (the checker on the host cores of the GPU
    machine finishes a tree of these sizes in 10 to 25 seconds)."""
    for t in trees:
        to, tg = ob.tree(t), model.tree(t)
        for key in ("fid", "quantized", "gain"):
            assert np.array_equal(to[key], tg[key]), (key, t)
        assert np.array_equal(to["weights"], tg["weights"], equal_nan=True), t
    if leaves:
        assert np.array_equal(ob.leaf(), model.leaves())
    assert np.array_equal(ob.yhat(), model.train_yhat())


@pytest.mark.timeout(900)
def test_configs2_full_size(arb, oracle):
    import bench
    rows, F, depth, eta, lam = 50_000_000, 200, 10, 0.3, 1.0
    bins, y = bench.make_config2_bins(rows, F)
    data = arb.DMatrix(bins, y=y, quantized=True)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 64, "double_precision": True},
           "tree": {"max_depth": depth, "eta": eta, "lambda": lam, "min_child_weight": 1.0, "min_leaf_size": 1}}
    model = arb.Garden(cfg, data)
    ob = oracle.Booster(bins, y=y, config=cfg, binned=True)
    model.grow_tree()
    ob.grow(1)
    _same_as_checker(ob, model, [0])
    before = model.train_yhat()
    model.grow_tree()
    ob.grow(1)
    _same_as_checker(ob, model, [1])
    del ob
    tree, leaf, after = model.tree(1), model.leaves(), model.train_yhat()
    assert (tree["quantized"] >= 0).sum() > 900, "not a full depth-10 tree"
    assert np.array_equal(leaf, _walk(tree, bins, depth)), "row -> leaf"
    g = y - before                                            # the gradient pass, in fp32 as on the device
    assert _check_leaf_weights(tree, leaf, g, np.ones_like(g), eta, lam) > 900
    assert np.array_equal(after, before + tree["weights"][leaf]), "prediction update"
    rng = np.random.default_rng(5)
    others = [int(f) for f in rng.choice(F, 7, replace=False)]
    _check_root_split(oracle, tree, bins, g, np.ones_like(g), 1, sorted(set([int(tree["fid"][0])] + others)), 65, lam)


@pytest.mark.timeout(900)
def test_configs3_full_size(arb, oracle):
    import bench
    rows, F, K, depth, eta, lam = 20_000_000, 100, 10, 6, 0.2, 1.0
    X, labels = bench.make_config3(rows, F, K)
    data = arb.DMatrix(X, labels=labels)
    cfg = {"objective": 4, "method": 1, "internals": {"hist_size": 256, "double_precision": True},
           "tree": {"max_depth": depth, "eta": eta, "lambda": lam, "min_child_weight": 1.0, "min_leaf_size": 1,
                    "labels_count": K}}
    model = arb.Garden(cfg, data)
    model.grow_tree()
    ob = oracle.Booster(X, labels=labels, config=cfg)      # the first round against the checker
    del X
    ob.grow(1)
    _same_as_checker(ob, model, range(K), leaves=False)
    del ob
    k = K - 1                                                 # the last tree of a round belongs to the last class
    start = model.train_yhat().reshape(K, rows).copy()        # the scores the second round starts from
    model.set_inspect(True)                                   # keeps the round's gradients for grad()
    model.grow_tree()
    tree, leaf = model.tree(2 * K - 1), model.leaves()
    after = model.train_yhat().reshape(K, rows)[k]
    g_all, h_all = model.grad()
    g, h = g_all[k * rows:(k + 1) * rows], h_all[k * rows:(k + 1) * rows]
    bins = data.bins()
    assert (tree["quantized"] >= 0).sum() == 63, "not a full depth-6 tree"
    assert np.array_equal(leaf, _walk(tree, bins, depth)), "row -> leaf"
    assert _check_leaf_weights(tree, leaf, g, h, eta, lam) == 64
    assert np.array_equal(after, start[k] + tree["weights"][leaf]), "prediction update"
    # the round's gradients: soft-max of the scores it started from (a sample of the rows, in float64)
    pick = np.random.default_rng(7).choice(rows, 200000, replace=False)
    z = start[:, pick].astype(np.float64)
    p = np.exp(z - z.max(axis=0))
    p /= p.sum(axis=0)
    onehot = (labels[pick][None, :] == np.arange(K)[:, None]).astype(np.float64)
    assert np.abs(g_all.reshape(K, rows)[:, pick] - (onehot - p)).max() < 1e-6
    assert np.abs(h_all.reshape(K, rows)[:, pick] - 2 * p * (1 - p)).max() < 1e-6
    rng = np.random.default_rng(6)
    others = [int(f) for f in rng.choice(F, 5, replace=False)]
    _check_root_split(oracle, tree, bins, g, h, 3, sorted(set([int(tree["fid"][0])] + others)), 256, lam)


@pytest.mark.timeout(900)
def test_configs4_streamed(arb, oracle):
    # the out-of-core shape as the benchmark runs it: 64 M x 128 bin ids (8.2 GB) in pinned host
    # memory in blocks of 4 M rows, half of them kept in device memory, the others streamed at every
    # level; logistic objective, max_depth 8
    import bench
    rows, F, depth, eta, lam = 64_000_000, 128, 8, 0.1, 1.0
    bins, y = bench.make_stream_workload(rows, F)
    cfg = bench.config(depth, 256)
    cfg["internals"].update({"upload_features": False, "stream_block_rows": 1 << 22,
                             "stream_resident_bytes": 8 * (1 << 22) * F + 4096})
    data = arb.DMatrix(bins, y=y, quantized=True)
    model = arb.Garden(cfg, data)
    ob = oracle.Booster(bins, y=y, config=cfg, binned=True)
    model.grow_tree()
    ob.grow(1)
    _same_as_checker(ob, model, [0])
    del ob
    assert model.stream_residency() == (8, 16)
    before = model.train_yhat()
    model.grow_tree()
    tree, leaf, after = model.tree(1), model.leaves(), model.train_yhat()
    assert (tree["quantized"] >= 0).sum() > 100, "a tree with few splits"   # labels come from a depth-6 tree
    assert np.array_equal(leaf, _walk(tree, bins, depth)), "row -> leaf"
    s = 1.0 / (1.0 + np.exp(-before.astype(np.float64)))
    g, h = y - s, s * (1.0 - s)
    assert _check_leaf_weights(tree, leaf, g, h, eta, lam) > 100
    assert np.array_equal(after, before + tree["weights"][leaf]), "prediction update"
    others = [int(f) for f in np.random.default_rng(8).choice(F, 5, replace=False)]
    _check_root_split(oracle, tree, bins, g, h, 3, sorted(set([int(tree["fid"][0])] + others)), 256, lam)
