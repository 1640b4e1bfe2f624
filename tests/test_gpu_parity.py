"""Parity of the HIP path (through the C-ABI) against the CPU checker and the
reference's golden vectors.  Needs an MI355X: run with `-m gpu`."""
import itertools
import json

import numpy as np
import pytest

from conftest import concrete_config, load_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


def make_data(n, F, objective, seed, nan_frac=0.0):
    rng = np.random.default_rng(seed)
    X = rng.normal(size=(n, F)).astype(np.float32)
    X[:, F // 2:] = np.round(X[:, F // 2:] * 4) / 4          # repeated values
    if nan_frac:
        X[rng.random((n, F)) < nan_frac] = np.nan
    w = rng.normal(size=F)
    s = np.nan_to_num(X) @ w / np.sqrt(F)
    if objective == 0:
        y = (s + 0.3 * rng.normal(size=n)).astype(np.float32)
    else:
        y = (rng.random(n) < 1 / (1 + np.exp(-2 * s))).astype(np.float32)
    return X, y


def assert_same_training(arb, oracle, X, y, cfg, rounds, check_hist=True):
    """Grows `rounds` trees on both sides and compares every intermediate."""
    D = cfg["tree"]["max_depth"] + 1
    ob = oracle.Booster(X, y=y, config=cfg)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    g.set_inspect(check_hist)
    hs = cfg["internals"]["hist_size"]
    for r in range(rounds):
        ob.grow(1)
        g.grow_tree()
        if r == 0:
            gb = data.bins()
            assert np.array_equal(gb, ob.bins().astype(gb.dtype)), "bins"
            for f in range(X.shape[1]):
                t0, s0 = ob.thresholds(f)
                t1, s1 = data.thresholds(f, hs)
                assert s0 == s1 and np.array_equal(t0, t1), "thresholds"
        if check_hist:
            og, oh = ob.grad()
            gg, gh = g.grad()
            assert np.array_equal(og, gg), "grad round %d" % r
            if cfg["objective"] != 0:
                assert np.array_equal(oh, gh), "hess round %d" % r
            assert g.shifts() == ob.shifts()
            for level in range(D - 1):
                ho = ob.level_hist(level)[:, :, :hs + 1, :]
                hg = g.level_hist(level)
                slots = hg.shape[2]
                if hs + 1 <= slots:
                    assert np.array_equal(hg[:, :, :hs + 1, :], ho), "hist level %d round %d" % (level, r)
                    assert not hg[:, :, hs + 1:, :].any()
                else:  # hist_size above 255 on columns with few distinct values: 8-bit bins
                    assert np.array_equal(hg, ho[:, :, :slots, :])
        to, tg = ob.tree(r), g.tree(r)
        assert np.array_equal(to["fid"], tg["fid"]), "fid round %d" % r
        assert np.array_equal(to["quantized"], tg["quantized"]), "bin round %d" % r
        assert np.array_equal(to["threshold"], tg["threshold"]), "threshold round %d" % r
        assert np.array_equal(to["gain"], tg["gain"]), "gain round %d" % r
        assert np.array_equal(to["weights"], tg["weights"], equal_nan=True), "weights round %d" % r  # empty leaf with lambda 0: 0/0
        assert np.array_equal(ob.leaf(), g.leaves()), "row->leaf round %d" % r
        assert np.array_equal(ob.yhat(), g.train_yhat()), "y_hat round %d" % r
    po, pg = ob.predict(X), g.predict(data)
    # NaN: a row with a missing value that reaches a leaf empty in training (0 / 0 with lambda 0)
    assert np.allclose(po, pg, rtol=0, atol=1e-6, equal_nan=True), "predictions"
    return ob, g


# ---------------------------------------------------------------- quantiser
@pytest.mark.parametrize("case", load_golden("quantiser.json"), ids=lambda c: c["name"])
def test_quantiser_reference_goldens(arb, case):
    # tests/cpp/test_datamatrix.cu:25-197 through the device sort + bin assignment
    x = np.array(case["x"], np.float32).reshape(-1, 1)
    data = arb.DMatrix(x)
    data.quantize(case["hist_size"])
    assert data.bins()[:, 0].tolist() == case["bins"]
    thr, size = data.thresholds(0, case["hist_size"])
    assert int(size).bit_length() == case["bits"]
    if case.get("first_threshold_inf"):
        assert np.isinf(thr[0])


def _columns_for_quantiser(n, rng):
    cols = [
        rng.normal(size=n),                                   # continuous
        np.exp(rng.normal(size=n)),                           # skewed
        rng.integers(0, 7, size=n).astype(np.float64),        # few distinct values
        np.round(rng.normal(size=n) * 20) / 20,               # many ties
        np.where(rng.random(n) < 0.3, np.nan, rng.random(n)), # 30 % NaN
        np.concatenate([np.arange(n // 20), np.full(n - n // 20 - n // 2, n // 20), n // 20 + 1 + np.arange(n // 2)]),  # gap rule
        rng.choice([-np.inf, -1.5, -0.0, 0.0, 2.0, np.inf], size=n),  # infinities and signed zeros
        np.full(n, 3.25),                                     # constant
        -np.abs(rng.normal(size=n)) * 1e-30,                  # tiny negatives
    ]
    return np.stack(cols, axis=1).astype(np.float32)


@pytest.mark.parametrize("n,hist_size", [(5000, 16), (70000, 255), (4097, 64), (300, 256), (9000, 3)])
def test_quantiser_matches_oracle(arb, oracle, n, hist_size):
    X = _columns_for_quantiser(n, np.random.default_rng(n))
    data = arb.DMatrix(X)
    data.quantize(hist_size)
    bins = data.bins()
    for f in range(X.shape[1]):
        thr_o, bins_o, size_o = oracle.quantize_column(X[:, f], hist_size)
        thr_g, size_g = data.thresholds(f, hist_size)
        assert size_g == size_o, f
        assert np.array_equal(thr_g, thr_o), f
        assert np.array_equal(bins[:, f], bins_o.astype(np.uint8)), f


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("dp", [True, False])
@pytest.mark.parametrize("trick", [True, False])
def test_training_matches_oracle(arb, oracle, objective, dp, trick):
    X, y = make_data(20000, 11, objective, seed=3, nan_frac=0.02)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 63, "double_precision": dp, "use_hist_subtraction_trick": trick},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0, "min_child_weight": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=3)


@pytest.mark.parametrize("objective", [0, 1])
def test_training_without_inspection(arb, oracle, objective):
    # inspection off: the last pass of a tree also writes the next round's gradients
    X, y = make_data(30000, 28, objective, seed=21, nan_frac=0.01)
    cfg = {"objective": objective, "method": 1, "internals": {"hist_size": 128, "double_precision": True},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=4, check_hist=False)


@pytest.mark.parametrize("inspect", [True, False])
@pytest.mark.parametrize("trick", [True, False])
def test_logistic_with_fractional_labels(arb, oracle, inspect, trick):
    # 0/1 labels let the builder carry (g, h) as one float per row; any other label value
    # takes the two-array path, which must give the same bits as the checker too
    X, y = make_data(30000, 13, 1, seed=31, nan_frac=0.01)
    y[::3] = 0.25
    y[1::7] = 0.5
    cfg = {"objective": 1, "method": 1,
           "internals": {"hist_size": 100, "double_precision": True, "use_hist_subtraction_trick": trick},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=4, check_hist=inspect)


@pytest.mark.parametrize("labels,shift_g", [((-1.0, 1.0), 28), ((0.0, 2.5), 28), ((-6.0, 0.5), 27)])
def test_logistic_with_labels_outside_0_1(arb, oracle, labels, shift_g):
    # g = y - sigmoid leaves [-1, 1] when a label does: the fixed-point scale follows the label
    # range (max(|ymin - 1|, |ymax|) = 2, 2.5, 7 here) instead of dropping such rows
    X, y = make_data(20000, 9, 1, seed=17)
    y = np.where(y > 0, labels[1], labels[0]).astype(np.float32)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 64, "double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=3)
    assert g.shifts() == (shift_g, 32)
    # no gradient was dropped: the root's integer total is the sum of the rows' fixed-point values
    gg, _ = g.grad()
    total = int(np.rint(gg.astype(np.float64) * 2.0 ** shift_g).sum())
    assert int(g.level_hist(0)[0, 0, :, 0].sum()) == total and total != 0


def test_heavy_tailed_regression_targets(arb, oracle):
    # five targets 2^21 times larger than the rest set the fixed-point scale of every row (7
    # fractional bits for the typical residual); the device must still equal the checker bit
    # for bit, and the checker's splits equal those of fp64 accumulation (CPU test)
    rng = np.random.default_rng(1)
    n, F = 20000, 8
    X = rng.normal(size=(n, F)).astype(np.float32)
    y = (X[:, 0] * 2 + np.sin(X[:, 1] * 3) + 0.1 * rng.normal(size=n)).astype(np.float32)
    y[rng.choice(n, 5, replace=False)] *= 2.0 ** 21
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 63, "double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0, "min_leaf_size": 50}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=4)
    assert g.shifts()[0] <= 8


@pytest.mark.parametrize("inspect", [True, False])
@pytest.mark.parametrize("eta", [30.0, 70.0, 1e4])
def test_logistic_with_saturated_predictions(arb, oracle, inspect, eta):
    # a huge learning rate drives the raw predictions past the range of exp (|x| > 88.8 and
    # > 104): the sigmoid saturates to 0 and 1, hessians vanish, leaf weights blow up.  The
    # device evaluates exp as straight-line code with the special cases selected at the end;
    # the checker branches first.  Both must give the same bits, predictions included.
    X, y = make_data(20000, 6, 1, seed=5)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 32, "double_precision": True},
           "tree": {"max_depth": 4, "eta": eta, "lambda": 1e-3, "min_child_weight": 0.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=4, check_hist=inspect)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    for _ in range(4):
        g.grow_tree()
    raw = g.train_yhat()
    assert np.abs(raw).max() > 104.0    # the case the test is about
    p = g.predict(data)
    assert np.isfinite(p).all() and p.min() == 0.0 and p.max() == 1.0


@pytest.mark.parametrize("n,F,depth", [(1, 3, 2), (65, 1, 1), (2049, 5, 3), (70000, 8, 4), (5000, 32, 5)])
def test_last_pass_feeds_next_root_histogram(arb, oracle, n, F, depth):
    # logistic, inspection off: the pass that assigns the leaves of a tree also
    # builds the root histogram of the next tree
    X, y = make_data(n, F, 1, seed=n + F)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 64, "double_precision": False},
           "tree": {"max_depth": depth, "eta": 0.5, "lambda": 1.0, "min_child_weight": 0.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=5, check_hist=False)


def test_inspection_switched_on_between_rounds(arb, oracle):
    X, y = make_data(20000, 12, 1, seed=77)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 255, "double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.4, "lambda": 1.0}}
    ob = oracle.Booster(X, y=y, config=cfg)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    for r in range(6):
        g.set_inspect(r in (2, 3))  # off, off, on, on, off, off
        ob.grow(1)
        g.grow_tree()
        to, tg = ob.tree(r), g.tree(r)
        for key in ("fid", "quantized", "threshold", "gain"):
            assert np.array_equal(to[key], tg[key]), "%s round %d" % (key, r)
        assert np.array_equal(to["weights"], tg["weights"], equal_nan=True)
        assert np.array_equal(ob.yhat(), g.train_yhat()), "y_hat round %d" % r
        if r in (2, 3):
            for level in range(5):
                assert np.array_equal(g.level_hist(level)[:, :, :256, :], ob.level_hist(level)[:, :, :256, :])


# ----------------------------------------------- streamed (out-of-core) bins
@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("trick", [True, False])
@pytest.mark.parametrize("block_rows", [64, 1000, 4096, 1 << 20])
def test_streamed_bins_match_oracle(arb, oracle, objective, trick, block_rows):
    # upload_features = false: bins stay in pinned host blocks and are copied in
    # block by block at every level (reference: garden.cu:603-604,
    # hist_tree_grower.cu:335-366); results must not depend on it.
    # stream_resident_bytes 0: no block is kept in device memory, every one is copied at every level
    X, y = make_data(9000, 11, objective, seed=13, nan_frac=0.02)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 63, "double_precision": True, "use_hist_subtraction_trick": trick,
                         "upload_features": False, "stream_block_rows": block_rows, "stream_resident_bytes": 0},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=3)
    assert g.stream_residency() == (0, (9000 + max(block_rows, 64) - 1) // max(block_rows, 64))
    assert_same_training(arb, oracle, X, y, cfg, rounds=3, check_hist=False)


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("resident_blocks", [0, 1, 5, 9, -1])
def test_partly_resident_equals_resident_equals_streamed(arb, oracle, objective, resident_blocks):
    # The reference keeps as many columns on the device as fit into 0.9 of the free memory and
    # streams the others (src/io/io.cu:496-507, src/core/garden.cu:296-347); here whole row blocks
    # are kept.  Whatever share is resident, the trees are the checker's (and so those of the
    # resident matrix and of the fully streamed one).
    n, F, block_rows = 40000, 20, 4096           # 10 blocks of 5 quads x 4096 rows x 4 bytes
    X, y = make_data(n, F, objective, seed=23, nan_frac=0.03)
    block_bytes = 5 * block_rows * 4
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 100, "double_precision": True, "upload_features": False,
                         "stream_block_rows": block_rows,
                         "stream_resident_bytes": -1 if resident_blocks < 0 else resident_blocks * block_bytes + 100},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=3)
    assert g.stream_residency() == (10 if resident_blocks < 0 else resident_blocks, 10)
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=4, check_hist=False)
    resident = dict(cfg, internals=dict(cfg["internals"], upload_features=True))
    r = arb.Garden(resident, arb.DMatrix(X, y=y))
    for t in range(4):
        r.grow_tree()
        for key in ("fid", "quantized", "threshold", "gain", "weights"):
            assert np.array_equal(r.tree(t)[key], g.tree(t)[key], equal_nan=True), (t, key)
    assert r.stream_residency() == (0, 0)


def test_streamed_wide_matrix_and_prequantised(arb, oracle):
    rng = np.random.default_rng(3)
    n, F = 20000, 50
    bins = rng.integers(0, 256, size=(n, F), dtype=np.uint8)
    y = (bins[:, 3].astype(np.int32) + bins[:, 40] > 250).astype(np.float32)
    cfg = {"objective": 1, "method": 1,
           "internals": {"hist_size": 256, "double_precision": False, "upload_features": False,
                         "stream_block_rows": 6000},
           "tree": {"max_depth": 4, "eta": 0.5, "lambda": 1.0}}
    ob = oracle.Booster(bins, y=y, config=cfg, binned=True)
    data = arb.DMatrix(bins, y=y, quantized=True)
    g = arb.Garden(cfg, data)
    for r in range(2):
        ob.grow(1)
        g.grow_tree()
        to, tg = ob.tree(r), g.tree(r)
        for key in ("fid", "quantized", "gain", "weights"):
            assert np.array_equal(to[key], tg[key], equal_nan=True), (key, r)
        assert np.array_equal(ob.leaf(), g.leaves())
    assert np.array_equal(data.bins(), bins)
    # host prediction walks the pinned blocks
    assert np.allclose(g.predict(data), ob.predict(bins.astype(np.float32)), atol=1e-6)


def test_training_255_bins_28_features(arb, oracle):
    X, y = make_data(60000, 28, 1, seed=11)
    cfg = {"objective": 1, "method": 1,
           "internals": {"hist_size": 255, "double_precision": True},
           "tree": {"max_depth": 8, "eta": 0.1, "lambda": 1.0, "min_child_weight": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2)


def test_training_many_features_uses_feature_groups(arb, oracle):
    # 50 features do not fit one workgroup's LDS in the (g,h) form: two launches
    X, y = make_data(9000, 50, 1, seed=5)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 31, "double_precision": False},
           "tree": {"max_depth": 4, "eta": 0.5, "lambda": 0.5}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2)


@pytest.mark.parametrize("in_place", [2, 1, False])
@pytest.mark.parametrize("objective,F,hist", [(0, 36, 100), (1, 33, 100), (0, 70, 100), (1, 44, 256), (0, 48, 256),
                                              (1, 47, 255)])
def test_quad_groups_of_wide_matrices(arb, oracle, objective, F, hist, in_place):
    # 33 and 36 features: a group of eight quads and a group of one; 70: three groups.  in_place 2:
    # rows stay where they are as records and (row id, gradients) are re-ordered; False: the fused
    # pass moves the rows once per group of quads; 1 (the default): whichever was measured faster
    # for the shape (in place from 48 features on, or when the bins in use fit one LDS histogram:
    # 44 and 47 features at 256 bins move their rows, 48 do not)
    X, y = make_data(20000, F, objective, seed=F, nan_frac=0.05)
    if hist >= 255:     # continuous columns, so that the features use all the bins
        X[:, F // 2:] = np.random.default_rng(F).normal(size=(20000, F - F // 2)).astype(np.float32)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": hist, "double_precision": True, "wide_rows_in_place": in_place},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2)


@pytest.mark.parametrize("trick", [True, False])
@pytest.mark.parametrize("n,F,depth,objective", [(1, 40, 3, 0), (63, 33, 4, 1), (4097, 130, 5, 1), (50000, 200, 7, 0), (3000, 300, 4, 0)])
def test_rows_in_place_shapes(arb, oracle, n, F, depth, objective, trick):
    # the records path on ragged row counts, record widths that are not a multiple of eight words,
    # with and without sibling subtraction, inspection on (histograms compared) and off
    X, y = make_data(n, F, objective, seed=n + F, nan_frac=0.02)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 63, "double_precision": True, "use_hist_subtraction_trick": trick},
           "tree": {"max_depth": depth, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2, check_hist=n < 10000)


@pytest.mark.parametrize("trick", [True, False])
@pytest.mark.parametrize("n,F,depth,objective,hist", [(4097, 100, 5, 1, 255), (20000, 33, 6, 0, 256),
                                                      (63, 130, 4, 1, 200), (30000, 70, 6, 1, 256)])
def test_rows_in_place_in_groups(arb, oracle, n, F, depth, objective, hist, trick):
    # histograms too large for one LDS: the records are read once per group of 32 features (one
    # or two 16-byte pieces per launch), 256 bins per feature; the last group holds fewer blocks
    X, y = make_data(n, F, objective, seed=n + F + 1, nan_frac=0.02)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": hist, "double_precision": True, "use_hist_subtraction_trick": trick},
           "tree": {"max_depth": depth, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2, check_hist=n < 10000)


def test_rows_in_place_thousand_features(arb, oracle):
    # 1000 features of at most 8 bins: records of 256 words, a wave reads one record at a time
    X, y = make_data(2000, 1000, 0, seed=1000, nan_frac=0.02)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 7, "double_precision": True},
           "tree": {"max_depth": 3, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2)


@pytest.mark.parametrize("objective", [0, 1])
def test_one_launch_records_leave_the_cells_of_unused_bins_zero(arb, oracle, objective):
    # 40 features whose bin ids stop at 64 under hist_size 256: every feature fits ONE LDS histogram of
    # the 65 bins in use, the slab reduction writes only those, and the split scan and the root totals
    # still read 256 cells per feature: the cells above the bins in use must be zero in every node
    # histogram of every level of every tree (they are cleared once, when the booster is created)
    rng = np.random.default_rng(40)
    n, F = 30000, 40
    bins = rng.integers(0, 65, size=(n, F), dtype=np.uint8)
    s = bins[:, 3].astype(np.float32) / 16 - (bins[:, 17] > 30) + (bins[:, 39] == 64) + 0.3 * rng.normal(size=n)
    y = s.astype(np.float32) if objective == 0 else (s > 1).astype(np.float32)
    cfg = {"objective": objective, "method": 1, "internals": {"hist_size": 256, "double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0}}
    ob = oracle.Booster(bins, y=y, config=cfg, binned=True)
    g = arb.Garden(cfg, arb.DMatrix(bins, y=y, quantized=True))
    g.set_inspect(True)
    for r in range(4):
        ob.grow(1)
        g.grow_tree()
        for level in range(5):
            hg, ho = g.level_hist(level), ob.level_hist(level)
            assert hg.shape[2] == 256
            assert np.array_equal(hg, ho[:, :, :256, :]), (r, level)
            assert not hg[:, :, 65:, :].any()
        for key in ("fid", "quantized", "gain", "weights"):
            assert np.array_equal(ob.tree(r)[key], g.tree(r)[key]), (r, key)
    assert np.array_equal(ob.yhat(), g.train_yhat())


def test_many_trees_without_reading_the_model(arb, oracle):
    # tree records wait on the device (a ring of 64) until the model is read
    X, y = make_data(3000, 6, 1, seed=64)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 32, "double_precision": True},
           "tree": {"max_depth": 3, "eta": 0.2, "lambda": 1.0}}
    rounds = 150
    ob = oracle.Booster(X, y=y, config=cfg)
    ob.grow(rounds)
    data = arb.DMatrix(X, y=y)
    g = arb.Garden(cfg, data)
    for _ in range(rounds):
        g.grow_tree()
    for r in range(rounds):
        to, tg = ob.tree(r), g.tree(r)
        for key in ("fid", "quantized", "threshold", "gain", "weights"):
            assert np.array_equal(to[key], tg[key], equal_nan=True), "%s of tree %d" % (key, r)
    assert np.array_equal(ob.yhat(), g.train_yhat())
    assert np.allclose(ob.predict(X), g.predict(data), rtol=0, atol=1e-6)


@pytest.mark.parametrize("depth,objective,trick,upload",
                         [(11, 1, True, True), (12, 0, True, True), (12, 1, False, True), (13, 1, True, True),
                          (11, 0, True, False)])
def test_deep_trees(arb, oracle, depth, objective, trick, upload):
    # up to 4096 nodes on the last level, most of them empty
    X, y = make_data(120000, 9, objective, seed=depth, nan_frac=0.01)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 64, "double_precision": True, "use_hist_subtraction_trick": trick,
                         "upload_features": upload, "stream_block_rows": 50000},
           "tree": {"max_depth": depth, "eta": 0.3, "lambda": 1.0, "min_child_weight": 0.0, "min_leaf_size": 0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2, check_hist=(depth <= 11))


@pytest.mark.parametrize("depth", [11, 12])
def test_deep_trees_on_28_features(arb, oracle, depth):
    # logistic, inspection off, 7 quads: the last pass keeps the 128 KB histogram of the next root,
    # the node table, the leaf weights and the exp table in LDS; at depth 11 they just fit (152 KB),
    # at depth 12 they do not and the pass runs without the histogram
    X, y = make_data(100000, 28, 1, seed=100 + depth, nan_frac=0.01)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 255, "double_precision": True},
           "tree": {"max_depth": depth, "eta": 0.3, "lambda": 1.0, "min_child_weight": 0.0, "min_leaf_size": 0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=3, check_hist=False)


def test_depth_limit_is_an_error(arb):
    X, y = make_data(1000, 3, 0, seed=1)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 16}, "tree": {"max_depth": 14}}
    with pytest.raises(Exception, match="unsupported depth"):
        arb.Garden(cfg, arb.DMatrix(X, y=y)).grow_tree()


@pytest.mark.parametrize("n", [1, 2, 63, 64, 65, 1023, 1025, 4097])
def test_ragged_row_counts(arb, oracle, n):
    X, y = make_data(n, 5, 0, seed=n)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 16, "double_precision": True},
           "tree": {"max_depth": 3, "eta": 1.0, "lambda": 0.0, "min_child_weight": 0, "min_leaf_size": 0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2)


def test_regularisation_and_guards(arb, oracle):
    X, y = make_data(5000, 6, 1, seed=8)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 40, "double_precision": False},
           "tree": {"max_depth": 6, "eta": 0.2, "lambda": 2.0, "alpha": 0.5, "min_child_weight": 20.0,
                    "min_leaf_size": 50, "gamma_absolute": 0.5, "gamma_relative": 0.001,
                    "max_leaf_weight": 0.3}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=3)


def test_max_depth_1(arb, oracle):
    X, y = make_data(3000, 4, 0, seed=2)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 255},
           "tree": {"max_depth": 1, "eta": 0.5, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=2)


# ------------------------------------------------------------ 16-bit bins
@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("trick", [True, False])
@pytest.mark.parametrize("hist_size,F", [(1000, 5), (300, 3), (4095, 2)])
def test_sixteen_bit_bins(arb, oracle, objective, trick, hist_size, F):
    # continuous columns with hist_size above 255 need more than 256 bin ids per feature
    X, y = make_data(30000, F, objective, seed=hist_size, nan_frac=0.02)
    X[:, : (F + 1) // 2] = np.random.default_rng(1).normal(size=(30000, (F + 1) // 2)).astype(np.float32)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": hist_size, "double_precision": True, "use_hist_subtraction_trick": trick},
           "tree": {"max_depth": 5, "eta": 0.4, "lambda": 1.0, "min_child_weight": 0.5}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=2)
    bits, slots = g.data.bin_layout()
    assert bits == 16 and slots >= hist_size + 1


def test_sixteen_bit_bins_without_inspection_and_limits(arb, oracle):
    X, y = make_data(9000, 4, 1, seed=5)
    X[:, 0] = np.random.default_rng(2).normal(size=9000).astype(np.float32)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 600, "double_precision": False},
           "tree": {"max_depth": 4, "eta": 0.3, "lambda": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=3, check_hist=False)
    too_many = dict(cfg, internals={"hist_size": 5000})
    with pytest.raises(Exception, match="hist_size above 4095"):
        arb.Garden(too_many, arb.DMatrix(X, y=y)).grow_tree()
    streamed = dict(cfg, internals={"hist_size": 600, "upload_features": False})
    with pytest.raises(Exception, match="16-bit bins are not built for streamed"):
        arb.Garden(streamed, arb.DMatrix(X, y=y)).grow_tree()


def _skewed_matrix(n, seed):
    """Columns whose rows pile up in one bin: 30 % missing, Zipf categories, a binary flag, zeros, a constant."""
    rng = np.random.default_rng(seed)
    X = rng.normal(size=(n, 13)).astype(np.float32)
    X[:, :4][rng.random((n, 4)) < 0.3] = np.nan
    X[:, 4:7] = np.minimum(rng.zipf(1.3, size=(n, 3)), 200).astype(np.float32)
    X[:, 7] = (rng.random(n) < 0.05).astype(np.float32)
    X[:, 8] = np.where(rng.random(n) < 0.9, 0.0, X[:, 8])
    X[:, 9] = 3.5
    X[:, 10] = np.nan
    s = np.nan_to_num(X[:, 0]) + (X[:, 4] > 2) - X[:, 7] + 0.5 * X[:, 11]
    y = (rng.random(n) < 1 / (1 + np.exp(-s))).astype(np.float32)
    return X, y


@pytest.mark.parametrize("upload", [True, False])
@pytest.mark.parametrize("objective", [0, 1])
def test_rows_concentrated_in_one_bin(arb, oracle, upload, objective):
    # exercises the LDS replicas of the most frequent bin of every feature
    X, y = _skewed_matrix(40000, seed=21)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 255, "double_precision": True, "upload_features": upload,
                         "stream_block_rows": 9000},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0, "min_child_weight": 1.0}}
    assert_same_training(arb, oracle, X, y, cfg, rounds=3)


def test_duplicate_features_tie_to_the_lowest_feature_id(arb, oracle):
    # equal gains across features: the lowest feature id wins (hist_tree_grower.cu:59-60)
    X, y = make_data(8000, 6, 1, seed=12)
    X[:, 4] = X[:, 1]
    X[:, 5] = X[:, 0]
    X = X[:, [5, 4, 2, 3, 1, 0]].copy()  # the duplicates come first
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 64, "double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=3)
    for r in range(3):
        fid = g.tree(r)["fid"]
        assert not np.isin(fid, [4, 5]).any(), "a duplicate with the higher id was chosen"


def test_constant_features_give_unsplit_nodes(arb, oracle):
    X = np.ones((500, 3), np.float32)
    y = np.arange(500, dtype=np.float32)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 8},
           "tree": {"max_depth": 3, "eta": 0.5, "lambda": 1.0}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=1)
    assert (g.tree(0)["quantized"] == -1).all()
    model = json.loads(g.dump())
    assert all(n["threshold"] is None for n in model["model"][0]["nodes"] if not n["leaf"])


@pytest.mark.parametrize("bytree,bylevel,seed", [(0.5, 1.0, 0), (1.0, 0.6, 3), (0.7, 0.7, 11)])
def test_column_sampling(arb, oracle, bytree, bylevel, seed):
    # same shuffle stream on both sides (std::shuffle + std::default_random_engine(seed),
    # src/core/garden.cu:87,126-165); parity with the reference's stream is unpinned
    X, y = make_data(8000, 12, 1, seed=6)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 32, "double_precision": True, "seed": seed},
           "tree": {"max_depth": 4, "eta": 0.3, "lambda": 1.0, "colsample_bytree": bytree,
                    "colsample_bylevel": bylevel}}
    ob, g = assert_same_training(arb, oracle, X, y, cfg, rounds=4, check_hist=False)
    used = set()
    for t in range(4):
        tr = g.tree(t)
        used |= set(tr["fid"][tr["quantized"] >= 0].tolist())
    assert len(used) > 1


def test_column_sampling_too_small_is_an_error(arb):
    X, y = make_data(100, 3, 0, seed=1)
    for tree in ({"colsample_bytree": 0.1}, {"colsample_bytree": 0.5, "colsample_bylevel": 0.5}):
        g = arb.Garden({"objective": 0, "method": 1, "tree": dict(tree, max_depth=2)}, arb.DMatrix(X, y=y))
        with pytest.raises(arb.ArboretumError, match="too small"):
            g.grow_tree()


def test_softmax_matches_oracle(arb, oracle):
    # Parity unpinned against the reference (its soft-max kernel is empty,
    # src/core/objective.cu:91-100); the oracle restates the formula left in the
    # comment at objective.cu:60-89 and the GPU must reproduce it bit for bit.
    rng = np.random.default_rng(4)
    n, F, K = 12000, 9, 3
    X = rng.normal(size=(n, F)).astype(np.float32)
    W = rng.normal(size=(F, K))
    labels = np.argmax(X @ W + rng.gumbel(size=(n, K)), axis=1).astype(np.uint8)
    cfg = {"objective": 4, "method": 1, "internals": {"hist_size": 64, "double_precision": True},
           "tree": {"max_depth": 4, "eta": 0.3, "lambda": 1.0, "labels_count": K}}
    ob = oracle.Booster(X, labels=labels, config=cfg)
    data = arb.DMatrix(X, labels=labels)
    assert data.labels_count == K
    g = arb.train(cfg, data, 0)
    g.set_inspect(True)
    for r in range(3):
        ob.grow(1)
        g.grow_tree()
        og, oh = ob.grad()
        gg, gh = g.grad()
        assert np.array_equal(og, gg) and np.array_equal(oh, gh), "gradients round %d" % r
        for k in range(K):
            to, tg = ob.tree(r * K + k), g.tree(r * K + k)
            for key in ("fid", "quantized", "threshold", "weights"):
                assert np.array_equal(to[key], tg[key]), (key, r, k)
        assert np.array_equal(ob.yhat(), g.train_yhat())
    po, pg = ob.predict(X), g.predict(data)
    assert pg.shape == (n, K) and np.allclose(po, pg, atol=1e-6)
    assert np.allclose(pg.sum(axis=1), 1.0, atol=1e-5)
    acc = (np.argmax(pg, axis=1) == labels).mean()
    assert acc > 0.45     # far above chance (1/3): the trees learn


@pytest.mark.parametrize("seed", range(8))
def test_softmax_random_configurations(arb, oracle, seed):
    # both soft-max objectives over drawn shapes: class counts, depths, bin counts, missing values,
    # resident and streamed bins, with and without sibling subtraction and inspection
    rng = np.random.default_rng(900 + seed)
    n = int(rng.choice([257, 3000, 20000]))
    F = int(rng.choice([2, 7, 28, 33]))
    K = int(rng.choice([2, 3, 7]))
    X = rng.normal(size=(n, F)).astype(np.float32)
    X[rng.random(X.shape) < 0.02] = np.nan
    W = rng.normal(size=(F, K))
    labels = np.argmax(np.nan_to_num(X) @ W + rng.gumbel(size=(n, K)), axis=1).astype(np.uint8)
    labels[:K] = np.arange(K, dtype=np.uint8)   # every class present
    cfg = {"objective": int(rng.choice([3, 4])), "method": 1,
           "internals": {"hist_size": int(rng.choice([16, 64, 255])), "double_precision": bool(rng.integers(0, 2)),
                         "use_hist_subtraction_trick": bool(rng.integers(0, 2)),
                         "upload_features": bool(rng.random() < 0.7), "stream_block_rows": 1000},
           "tree": {"max_depth": int(rng.integers(1, 6)), "eta": 0.3, "lambda": float(rng.choice([0.5, 1.0])),
                    "min_child_weight": float(rng.choice([0.0, 1.0])), "labels_count": K}}
    ob = oracle.Booster(X, labels=labels, config=cfg)
    data = arb.DMatrix(X, labels=labels)
    g = arb.Garden(cfg, data)
    g.set_inspect(bool(seed & 1))
    for r in range(3):
        ob.grow(1)
        g.grow_tree()
        for k in range(K):
            to, tg = ob.tree(r * K + k), g.tree(r * K + k)
            for key in ("fid", "quantized", "threshold", "gain", "weights"):
                assert np.array_equal(to[key], tg[key], equal_nan=True), (key, r, k)
        assert np.array_equal(ob.yhat(), g.train_yhat()), "y_hat round %d" % r
    assert np.allclose(ob.predict(X), g.predict(data), rtol=0, atol=1e-6, equal_nan=True)


# ------------------------------------------------------ reference goldens
def _golden_cases(arb, fixture, X, y):
    for name, case in fixture["cases"].items():
        for dp, trick, upload in itertools.product([True, False], repeat=3):
            cfg = concrete_config(fixture["config"], double_precision=dp, use_hist_trick=trick,
                                  upload_features=upload, depth=case["max_depth"])
            data = arb.DMatrix(X, y=y)
            model = arb.train(cfg, data, case["trees"])
            per_tree = isinstance(case["true_values"][0], list)
            want = case["true_values"] if per_tree else [case["true_values"]]
            rounds = range(case["trees"]) if per_tree else [case["trees"] - 1]
            for i, w in zip(rounds, want):
                pred = model.predict(data, i + 1)
                assert np.allclose(pred, w), (name, dp, trick, upload, i)
            dumped = model.dump()
            created = json.loads(dumped)
            true = case["true_model"]
            assert len(true["model"]) == len(created["model"])
            for tt, ct in zip(true["model"], created["model"]):
                assert np.allclose(tt["weights"], ct["weights"], rtol=1e-4, atol=1e-6), name
                assert tt["nodes"] == ct["nodes"], (name, dp, trick, upload)
            loaded = arb.load(dumped)
            for i, w in zip(rounds, want):
                assert np.allclose(loaded.predict(data, i + 1), w)


def test_golden_hist_regression(arb):
    fx = load_golden("hist_regression_boston10.json")
    _golden_cases(arb, fx, np.array(fx["X"], np.float32), np.array(fx["y"], np.float32))


def test_golden_hist_logistic(arb):
    fx = load_golden("hist_logistic_iris.json")
    _golden_cases(arb, fx, np.array(fx["X"], np.float32),
                  (np.array(fx["target"]) != 2).astype(np.float32))


@pytest.mark.parametrize("hist_size", [12, 15, 16, 31, 32, 63, 64, 127, 128, 255, 256, 511, 512, 1023])
def test_sklearn_regressor_golden(arb, hist_size):
    # tests/py/test_sklearn_regressor.py:9-40 of the reference (hist method)
    fx = load_golden("hist_regression_boston10.json")
    X, y = np.array(fx["X"], np.float32), np.array(fx["y"], np.float32)
    want = fx["cases"]["test_single_tree_depth_1"]["true_values"][0]
    for dp in (True, False):
        m = arb.ArboretumRegression(max_depth=1, learning_rate=0.99999, n_estimators=1, verbosity=0,
                                    min_child_weight=1.0, min_leaf_size=1, colsample_bytree=1.0, l1=0, l2=0,
                                    double_precision=dp, method='hist', hist_size=hist_size)
        m.fit(arb.DMatrix(X, y=y), y)
        assert np.allclose(m.predict(arb.DMatrix(X)), want)
