"""The headline size (10.5 M rows x 28 features, 256 bins, max_depth 8, logistic): the HIP path
against the CPU checker bit for bit (three trees: splits, gains, leaf weights, every row's leaf,
y_hat, the first tree's histograms at every level), against itself along independent code paths
and against invariants of the algorithm."""
import os
import sys

import numpy as np
import pytest

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))

pytestmark = pytest.mark.gpu

ROWS, FEATURES, ROUNDS = 10_500_000, 28, 3


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


@pytest.fixture(scope="module")
def workload():
    import bench
    return bench.make_workload(ROWS, FEATURES)


def _config(trick=True, upload=True):
    import bench
    cfg = bench.config(8, 256)
    cfg["internals"]["use_hist_subtraction_trick"] = trick
    cfg["internals"]["upload_features"] = upload
    cfg["internals"]["stream_block_rows"] = 1 << 22
    return cfg


def _grow(arb, workload, cfg, inspect_first=False):
    X, y = workload
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    hists = None
    for r in range(ROUNDS):
        g.set_inspect(inspect_first and r == 0)
        g.grow_tree()
        if inspect_first and r == 0:
            hists = [g.level_hist(level) for level in range(8)]
    trees = [g.tree(r) for r in range(ROUNDS)]
    return {"garden": g, "data": data, "trees": trees, "yhat": g.train_yhat(), "leaves": g.leaves(), "hists": hists}


@pytest.fixture(scope="module")
def fused(arb, workload):
    # sibling subtraction on: fused partition + histogram passes; the first boosting round with inspection
    return _grow(arb, workload, _config(), inspect_first=True)


def _same_trees(a, b):
    for r in range(ROUNDS):
        for key in ("fid", "quantized", "threshold", "gain"):
            assert np.array_equal(a["trees"][r][key], b["trees"][r][key]), "%s of tree %d" % (key, r)
        assert np.array_equal(a["trees"][r]["weights"], b["trees"][r]["weights"], equal_nan=True), "weights of tree %d" % r
    assert np.array_equal(a["yhat"], b["yhat"])
    assert np.array_equal(a["leaves"], b["leaves"])


def test_histogram_invariants(fused):
    hists = fused["hists"]
    root = hists[0][0]                         # [F][256][3]
    totals = root.sum(axis=1)                  # per feature (sum g_q, sum h_q, count)
    assert (totals[:, 2] == ROWS).all()
    assert (totals == totals[0]).all(), "every feature's histogram adds up to the same node totals"
    for level in range(1, 8):
        h = hists[level]                       # [nodes][F][256][3]
        per_node = h.sum(axis=2)               # [nodes][F][3]
        assert (per_node == per_node[:, :1, :]).all(), "level %d: features disagree on node totals" % level
        parents = hists[level - 1].sum(axis=2)[:, 0, :]
        children = per_node[:, 0, :]
        assert np.array_equal(children[0::2] + children[1::2], parents), "level %d: children do not add up" % level
        # cell by cell: the two children of a node split its histogram between them
        assert np.array_equal(h[0::2] + h[1::2], hists[level - 1]), "level %d: cells do not add up" % level


def test_leaves_and_trees_are_consistent(fused):
    leaves = fused["leaves"]
    counts = np.bincount(leaves, minlength=256)
    assert counts.sum() == ROWS and len(counts) == 256
    # the counts of the last level's histograms are the leaf sizes of tree 0 only; for the last tree
    # check the weights: leaves that hold rows have finite weights
    w = fused["trees"][ROUNDS - 1]["weights"]
    assert np.isfinite(w[counts > 0]).all()


def test_device_predictions_match_host_walk_on_raw_floats(fused):
    # y_hat kept on the device (tree walks on bins) against the host prediction (walks on the raw
    # floats with the thresholds): bins, thresholds, leaf ids and weights must all agree
    g, data = fused["garden"], fused["data"]
    host = g.predict(data)
    dev = 1.0 / (1.0 + np.exp(-fused["yhat"].astype(np.float64)))
    assert np.abs(host - dev).max() < 1e-4


def test_without_sibling_subtraction_same_trees(arb, workload, fused):
    # un-fused path: stand-alone partition, both children built directly
    _same_trees(fused, _grow(arb, workload, _config(trick=False)))


def test_streamed_bins_same_trees(arb, workload, fused):
    # bins in pinned host memory, three 4 M-row blocks per level
    _same_trees(fused, _grow(arb, workload, _config(upload=False)))


def test_second_run_is_bit_identical(arb, workload, fused):
    _same_trees(fused, _grow(arb, workload, _config()))


def test_headline_config_bit_exact_against_the_checker(arb, workload, fused, oracle):
    # BASELINE configs[1] at its full size: same seeded input on both sides
    X, y = workload
    ob = oracle.Booster(X, y=y, config=_config(), threads=16)
    ob.grow(1)
    for level in range(8):      # the first tree's integer histograms, every node of every level
        ho = ob.level_hist(level)
        hg = fused["hists"][level]
        assert np.array_equal(hg, ho[:, :, :hg.shape[2], :]), "histograms of level %d" % level
        assert not ho[:, :, hg.shape[2]:, :].any()
    ob.grow(ROUNDS - 1)
    for r in range(ROUNDS):
        to, tg = ob.tree(r), fused["trees"][r]
        for key in ("fid", "quantized", "threshold", "gain"):
            assert np.array_equal(to[key], tg[key]), "%s of tree %d" % (key, r)
        assert np.array_equal(to["weights"], tg["weights"], equal_nan=True), "leaf weights of tree %d" % r
        assert (tg["quantized"] >= 0).sum() > 200, "tree %d is not a full depth-8 tree" % r
    assert np.array_equal(ob.leaf(), fused["leaves"]), "row -> leaf of the last tree"
    assert np.array_equal(ob.yhat(), fused["yhat"]), "y_hat after %d trees" % ROUNDS
    po = ob.predict(X)
    pg = fused["garden"].predict(fused["data"])
    assert np.abs(po - pg).max() < 1e-4
