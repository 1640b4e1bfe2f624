"""Pins the CPU checker against every golden vector the reference's own tests
hold for the histogram path (no GPU needed)."""
import itertools
import math

import numpy as np
import pytest

from conftest import check_hist_sum, concrete_config, hist_sum_inputs, load_golden


# ---------------------------------------------------------------- quantiser
@pytest.mark.parametrize("case", load_golden("quantiser.json"), ids=lambda c: c["name"])
def test_quantiser_golden(oracle, case):
    thr, bins, size = oracle.quantize_column(np.array(case["x"], np.float32), case["hist_size"])
    assert bins.tolist() == case["bins"]
    assert int(size).bit_length() == case["bits"]          # io.cu:411: 32 - clz(size)
    if case.get("first_threshold_inf"):
        assert np.isinf(thr[0])


def test_quantiser_midpoints_when_rows_fit(oracle):
    # rows <= hist_size: thresholds are the midpoints of consecutive distinct values
    x = np.array([3.0, 1.0, 2.0, 2.0, 7.5, -1.0], np.float32)
    thr, bins, size = oracle.quantize_column(x, 16)
    u = np.unique(x)
    assert size == len(u)
    assert np.array_equal(thr[:size - 1], ((u[1:] + u[:-1]) * 0.5).astype(np.float32))
    assert np.array_equal(bins, np.searchsorted(u, x))


def test_quantiser_nan_goes_to_bin_size(oracle):
    x = np.array([0.0, np.nan, 1.0, 2.0, np.nan, 3.0], np.float32)
    thr, bins, size = oracle.quantize_column(x, 8)
    assert size == 4
    assert bins.tolist() == [0, 4, 1, 2, 4, 3]


def test_quantiser_gap_drops_trailing(oracle):
    # 100 distinct, then 1000 equal, then 900 distinct with B = 20: everything
    # after the first unset threshold is dropped (io.cu:403-408)
    x = np.concatenate([np.arange(100), np.full(1000, 100.0), 101 + np.arange(900)]).astype(np.float32)
    thr, bins, size = oracle.quantize_column(x, 20)
    assert size == 2
    assert bins.max() == 1


# ------------------------------------------------------------ gain / arg-max
def _scan(oracle, kind, bins, g, h, B, params):
    mls, mcw, ga, gr, lam, alpha = params
    G = np.zeros(B)
    H = np.zeros(B)
    C = np.zeros(B, np.int64)
    for b_, g_, h_ in zip(bins, g, h):
        G[b_] += g_
        H[b_] += h_
        C[b_] += 1
    best, bg = -1, 0.0
    gains = []
    for b_ in range(B):
        gl, hl, cl = G[:b_ + 1].sum(), H[:b_ + 1].sum(), int(C[:b_ + 1].sum())
        v = oracle.lib().orc_gain(kind, gl, hl, cl, G.sum(), H.sum(), int(C.sum()), mls, mcw, ga, gr,
                                  lam, alpha, 0.0)
        gains.append(v)
        if v > 0 and v >= bg:
            best, bg = b_, v
    return best, bg, G, gains


@pytest.mark.parametrize("case", load_golden("gain.json"), ids=lambda c: c["name"])
@pytest.mark.parametrize("kind", [2, 3])
def test_gain_golden(oracle, case, kind):
    for node in case["nodes"]:
        best, bg, G, _ = _scan(oracle, kind, node["bins"], node["g"], node["h"], case["hist_size"],
                               case["params"])
        assert best == node["best_bin"]
        assert bg == pytest.approx(node["gain"], rel=4e-7)   # ASSERT_FLOAT_EQ: 4 ulp
        if "sums" in node:
            assert G.tolist() == node["sums"]


@pytest.mark.parametrize("kind", [0, 1, 2, 3])
def test_gain_closed_form(oracle, kind):
    # alpha = 0: side gain = G^2/(H+lambda); gain = GL^2/(HL+l) + GR^2/(HR+l) - GT^2/(HT+l)
    rng = np.random.default_rng(1)
    for _ in range(200):
        cl, cr = int(rng.integers(1, 50)), int(rng.integers(1, 50))
        gl, gr = rng.normal() * cl, rng.normal() * cr
        if kind < 2:
            hl, hr = float(cl), float(cr)
        else:
            hl, hr = rng.uniform(0.5, 1) * cl, rng.uniform(0.5, 1) * cr
        lam = float(rng.uniform(0, 2))
        v = oracle.lib().orc_gain(kind, gl, hl, cl, gl + gr, hl + hr, cl + cr, 1, 0.0, 0.0, 0.0, lam,
                                  0.0, 0.0)
        ref = gl * gl / (hl + lam) + gr * gr / (hr + lam) - (gl + gr) ** 2 / (hl + hr + lam)
        assert v == pytest.approx(max(ref, 0.0), rel=2e-4, abs=1e-4)


def test_gain_guards(oracle):
    g = oracle.lib().orc_gain
    # min_leaf_size on either side
    assert g(2, 1.0, 1.0, 1, 3.0, 4.0, 4, 2, 0.0, 0, 0, 1.0, 0, 0) == 0.0
    # min_child_weight on |H| (pair form only, gain.cu:160-162)
    assert g(2, 1.0, 0.5, 5, -3.0, 4.0, 10, 1, 1.0, 0, 0, 1.0, 0, 0) == 0.0
    assert g(0, 1.0, 0.0, 5, -3.0, 0.0, 10, 1, 100.0, 0, 0, 1.0, 0, 0) == 0.0  # weights forced to 0
    # gamma_absolute
    v = g(2, 4.0, 2.0, 2, 0.0, 4.0, 4, 1, 0.0, 0, 0, 0.0, 0, 0)
    assert v == pytest.approx(16.0)
    assert g(2, 4.0, 2.0, 2, 0.0, 4.0, 4, 1, 0.0, 16.0, 0, 0.0, 0, 0) == 0.0
    # L1: |G| <= alpha gives weight 0
    assert oracle.lib().orc_weight(2, 0.5, 2.0, 3, 1, 0.0, 1.0, 0.75, 0.0) == 0.0
    assert oracle.lib().orc_weight(2, -2.0, 2.0, 3, 1, 0.0, 1.0, 0.5, 0.0) == pytest.approx(-0.5)
    assert oracle.lib().orc_weight(2, -20.0, 2.0, 3, 1, 0.0, 1.0, 0.5, 1.5) == -1.5   # max_leaf_weight


# ---------------------------------------------------------------- histograms
@pytest.mark.parametrize("case", load_golden("hist_sum.json"), ids=lambda c: c["name"])
def test_hist_sum_golden(oracle, case):
    bins, g, offs = hist_sum_inputs(case)
    n, H = case["rows"], case["hist_size"]
    shift = oracle.lib().orc_fix_shift(float(g.max()))
    rows = np.arange(n)
    nodes = len(offs) - 1
    hists = [oracle.hist_fixed_u8(bins, g, None, shift, 0, sel=(rows >= offs[k]) & (rows < offs[k + 1]))[0]
             for k in range(nodes)]
    if case["trick"]:
        # only the smaller sibling is accumulated (ties -> left, hist_grad_sum.cu:279-294); the
        # other one is the parent the test passes in minus it
        for k in range(0, nodes, 2):
            par = np.zeros_like(hists[k])
            par[:H, 0] = np.array(case["parent_sum"]) * 2.0 ** shift
            par[:H, 2] = case["parent_count"]
            left_built = offs[k + 1] - offs[k] <= offs[k + 2] - offs[k + 1]
            derived = par - hists[k if left_built else k + 1]
            # sibling subtraction is exact on the integers
            assert np.array_equal(derived, hists[k + 1 if left_built else k])
            hists[k + 1 if left_built else k] = derived
    count = [h[:, 2] for h in hists]
    total = [h[:, 0] * 2.0 ** -shift for h in hists]
    check_hist_sum(case, count, total)


def test_fixed_point_scale(oracle):
    L = oracle.lib()
    assert L.orc_fix_shift(1.0) == 29 and L.orc_fix_shift(0.99) == 30 and L.orc_fix_shift(0.0) == 30
    assert L.orc_to_fixed(1.0, 30) == 1 << 30
    assert L.orc_to_fixed(-0.25, 32) == -(1 << 30)
    assert L.orc_to_fixed(float("nan"), 30) == 0


def test_expf_within_one_ulp_of_libm(oracle):
    xs = np.concatenate([np.linspace(-100, 88, 20001), np.random.default_rng(0).normal(size=20000) * 5])
    xs = xs.astype(np.float32)
    ours = np.array([oracle.lib().orc_expf(float(x)) for x in xs], np.float32)
    ref = np.exp(xs.astype(np.float64))
    ok = np.isfinite(ref) & (ref > 1e-37)
    ulp = np.spacing(ref[ok].astype(np.float32)).astype(np.float64)
    assert np.all(np.abs(ours[ok].astype(np.float64) - ref[ok]) <= 0.5000001 * ulp + 0)


# ------------------------------------------------- end-to-end golden models
def _run_cases(oracle, fixture, X, y):
    combos = list(itertools.product([True, False], repeat=3))
    for name, case in fixture["cases"].items():
        for dp, trick, upload in combos:
            for accum in (0, 1):
                cfg = concrete_config(fixture["config"], double_precision=dp, use_hist_trick=trick,
                                      upload_features=upload, depth=case["max_depth"])
                b = oracle.Booster(X, y=y, config=cfg, accum=accum)
                b.grow(case["trees"])
                if isinstance(case["true_values"][0], list):   # predictions after every tree
                    for i in range(case["trees"]):
                        pred = b.predict(X, i + 1)
                        assert np.allclose(pred, case["true_values"][i]), (name, dp, trick, accum, i)
                else:                                           # predictions of the whole model
                    assert np.allclose(b.predict(X), case["true_values"]), (name, dp, trick, accum)
                model = b.model_dict()
                true = case["true_model"]["model"]
                assert len(true) == len(model["model"])
                for tt, ct in zip(true, model["model"]):
                    assert np.allclose(tt["weights"], ct["weights"], rtol=1e-4, atol=1e-6), name
                    assert tt["nodes"] == ct["nodes"], (name, dp, trick, accum)


def test_golden_exact_regression_boston(oracle):
    # method 0 (exact): tests/py/test_regression.py of the reference
    fx = load_golden("exact_regression_boston10.json")
    _run_cases(oracle, fx, np.array(fx["X"], np.float32), np.array(fx["y"], np.float32))


def test_golden_exact_logistic_iris(oracle):
    # method 0 (exact): tests/py/test_logresression.py of the reference
    fx = load_golden("exact_logistic_iris.json")
    _run_cases(oracle, fx, np.array(fx["X"], np.float32), (np.array(fx["target"]) != 2).astype(np.float32))


def _brute_force_exact_root(oracle, X, g, h, kind, params):
    """The reference's exact split search (continuous_tree_grower.cu:9-49) on one node, in plain
    Python: per feature sort the rows by value, exclusive prefix sums, the gain at every position
    where the value changes, best gain with ties to the highest position, then to the lowest
    feature.  Returns (feature, threshold value, gain)."""
    mls, mcw, ga, gr, lam, alpha = params
    n, F = X.shape
    GT, HT = float(np.sum(g.astype(np.float64))), float(np.sum(h.astype(np.float64)))
    best = (-1, None, 0.0)
    for f in range(F):
        order = np.argsort(X[:, f], kind="stable")
        xs, gs, hs = X[order, f], g[order].astype(np.float64), h[order].astype(np.float64)
        cg, ci = 0.0, -1
        for i in range(1, n):
            if xs[i] != xs[i - 1]:
                gain = oracle.lib().orc_gain(kind, float(gs[:i].sum()), float(hs[:i].sum()), i, GT, HT, n, mls,
                                             mcw, ga, gr, lam, alpha, 0.0)
                if gain > 0 and gain >= cg:
                    cg, ci = gain, i
        if ci >= 0 and (best[0] < 0 or cg > best[2]):
            best = (f, float(xs[ci]), cg)
    return best


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("seed", range(6))
def test_exact_root_split_against_brute_force(oracle, objective, seed):
    rng = np.random.default_rng(100 + seed)
    n, F = 60, 4
    X = np.round(rng.normal(size=(n, F)) * 3).astype(np.float32) / 2      # many repeated values
    X[:, 1] = rng.normal(size=n).astype(np.float32)                       # and one all-distinct column
    y = (X[:, 0] + X[:, 1] > 0).astype(np.float32) if objective else (X[:, 0] * 2 + rng.normal(size=n)).astype(np.float32)
    cfg = {"objective": objective, "method": 0, "internals": {"double_precision": True},
           "tree": {"max_depth": 1, "eta": 1.0, "lambda": 0.5, "min_child_weight": 0.0, "min_leaf_size": 1,
                    "initial_y": 0.5}}
    b = oracle.Booster(X, y=y, config=cfg, accum=1)
    b.grow(1)
    g, h = b.grad()
    if objective == 0:
        h = np.ones_like(g)
    f, thr, gain = _brute_force_exact_root(oracle, X, g, h, 1 if objective == 0 else 3, (1, 0.0, 0.0, 0.0, 0.5, 0.0))
    t = b.tree(0)
    assert f >= 0 and t["fid"][0] == f
    assert t["threshold"][0] == np.float32(thr)           # the smallest value that goes right
    assert t["gain"][0] == pytest.approx(gain, rel=1e-6)
    # the rows: value < threshold left, as prediction walks them
    assert np.array_equal(b.leaf(), (X[:, f] >= thr).astype(np.uint32))


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("accum", [0, 1])
def test_exact_mode_with_ranks_beyond_16_bits(oracle, objective, accum):
    # More than 65535 distinct values in a feature: the checker keeps 32-bit ranks.  Nothing else
    # of the exact mode differs, so with the switch that forces that branch the trees, leaves and
    # predictions are those of the 16-bit ranks (which the goldens and the brute force above pin).
    rng = np.random.default_rng(77 + objective)
    n, F = 3000, 4
    X = rng.normal(size=(n, F)).astype(np.float32)
    X[:, 2] = np.round(X[:, 2], 1)
    y = (X[:, 0] + X[:, 2] > 0).astype(np.float32) if objective else (X[:, 0] * 2 + rng.normal(size=n)).astype(np.float32)
    cfg = {"objective": objective, "method": 0, "internals": {"double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.5, "lambda": 1.0, "min_child_weight": 1.0}}
    grown = []
    try:
        for wide in (False, True):
            oracle.force_wide_ranks(wide)
            b = oracle.Booster(X, y=y, config=cfg, accum=accum)
            b.grow(3)
            grown.append(([b.tree(t) for t in range(3)], b.leaf(), b.yhat(), b.predict(X)))
    finally:
        oracle.force_wide_ranks(False)
    for ta, tb in zip(grown[0][0], grown[1][0]):
        for key in ta:
            assert np.array_equal(ta[key], tb[key], equal_nan=True), key
    assert (grown[0][0][2]["quantized"] >= 0).sum() > 20
    for k in (1, 2, 3):
        assert np.array_equal(grown[0][k], grown[1][k])


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("seed", range(6))
def test_hist_root_split_against_brute_force(oracle, objective, seed):
    # The histogram method chooses among the bins what the exact search chooses among the values
    # when the bin ids are taken as the values: left of a candidate are the rows of the bins up to
    # it, equal gains go to the highest bin (empty bins included, so the winner is the bin just
    # below the first bin that goes right), then to the lowest feature; NaN sits in the last bin
    # and always goes right.
    rng = np.random.default_rng(300 + seed)
    n, F = 80, 5
    X = np.round(rng.normal(size=(n, F)) * 2).astype(np.float32)          # few distinct values: empty bins
    X[:, 2] = rng.normal(size=n).astype(np.float32)
    X[rng.random((n, F)) < 0.1] = np.nan
    s = np.nan_to_num(X[:, 0]) + np.nan_to_num(X[:, 2])
    y = (s > 0).astype(np.float32) if objective else (2 * s + rng.normal(size=n)).astype(np.float32)
    cfg = {"objective": objective, "method": 1, "internals": {"hist_size": 16, "double_precision": True},
           "tree": {"max_depth": 1, "eta": 1.0, "lambda": 0.5, "min_child_weight": 0.0, "min_leaf_size": 1,
                    "initial_y": 0.5}}
    b = oracle.Booster(X, y=y, config=cfg, accum=1)
    b.grow(1)
    g, h = b.grad()
    if objective == 0:
        h = np.ones_like(g)
    bins = b.bins().astype(np.float32)
    f, first_right, gain = _brute_force_exact_root(oracle, bins, g, h, 1 if objective == 0 else 3,
                                                   (1, 0.0, 0.0, 0.0, 0.5, 0.0))
    t = b.tree(0)
    assert f >= 0 and t["fid"][0] == f
    assert t["quantized"][0] == int(first_right) - 1
    assert t["gain"][0] == pytest.approx(gain, rel=1e-6)
    assert np.array_equal(b.leaf(), (bins[:, f] >= first_right).astype(np.uint32))
    # the threshold reported is the one prediction needs: raw values below it are the left rows
    thr = t["threshold"][0]
    assert np.array_equal(X[:, f] < thr, bins[:, f] < first_right)


@pytest.mark.parametrize("objective", [0, 1])
@pytest.mark.parametrize("seed", range(4))
def test_hist_tree_against_node_by_node_brute_force(oracle, objective, seed):
    # A whole tree of depth 3, node by node in heap order: every node's split from the brute-force
    # search over its own rows, rows below the first right bin to child 2i+1 (left) and the others
    # to 2i+2, an unsplit or empty node sends everything left and is recorded as fid 0 / bin -1,
    # leaf weight = eta * G / (H + lambda) of the leaf's rows (H = row count for squared error).
    rng = np.random.default_rng(400 + seed)
    n, F, depth, lam, eta = 120, 4, 3, 0.5, 0.7
    X = np.round(rng.normal(size=(n, F)) * 2).astype(np.float32)
    X[:, 1] = rng.normal(size=n).astype(np.float32)
    s = X[:, 0] - X[:, 1] * X[:, 2]
    y = (s > 0).astype(np.float32) if objective else (s + 0.3 * rng.normal(size=n)).astype(np.float32)
    cfg = {"objective": objective, "method": 1, "internals": {"hist_size": 12, "double_precision": True},
           "tree": {"max_depth": depth, "eta": eta, "lambda": lam, "min_child_weight": 0.0, "min_leaf_size": 1,
                    "initial_y": 0.5}}
    b = oracle.Booster(X, y=y, config=cfg, accum=1)
    b.grow(1)
    g, h = b.grad()
    if objective == 0:
        h = np.ones_like(g)
    bins = b.bins().astype(np.float32)
    t = b.tree(0)
    rows = {0: np.arange(n)}
    for i in range((1 << depth) - 1):
        r = rows[i]
        f, first_right = -1, None
        if len(r) > 1:
            f, first_right, gain = _brute_force_exact_root(oracle, bins[r], g[r], h[r], 1 if objective == 0 else 3,
                                                           (1, 0.0, 0.0, 0.0, lam, 0.0))
        if f >= 0:
            assert (t["fid"][i], t["quantized"][i]) == (f, int(first_right) - 1), "node %d" % i
            assert t["gain"][i] == pytest.approx(gain, rel=1e-5)
            right = bins[r, f] >= first_right
        else:
            assert t["quantized"][i] == -1 and t["fid"][i] == 0 and np.isinf(t["threshold"][i]), "node %d" % i
            right = np.zeros(len(r), bool)
        rows[2 * i + 1], rows[2 * i + 2] = r[~right], r[right]
    first_leaf = (1 << depth) - 1
    leaf = np.empty(n, np.uint32)
    for k in range(1 << depth):
        r = rows[first_leaf + k]
        leaf[r] = k
        if len(r):
            G, H = g[r].astype(np.float64).sum(), h[r].astype(np.float64).sum()
            assert t["weights"][k] == pytest.approx(eta * G / (H + lam), rel=1e-5, abs=1e-7), "leaf %d" % k
    assert np.array_equal(b.leaf(), leaf)


def test_golden_regression_boston(oracle):
    fx = load_golden("hist_regression_boston10.json")
    _run_cases(oracle, fx, np.array(fx["X"], np.float32), np.array(fx["y"], np.float32))


def test_golden_logistic_iris(oracle):
    fx = load_golden("hist_logistic_iris.json")
    X = np.array(fx["X"], np.float32)
    y = (np.array(fx["target"]) != 2).astype(np.float32)
    _run_cases(oracle, fx, X, y)


# ------------------------------------------------------------- invariants
@pytest.mark.parametrize("objective", [0, 1])
def test_invariants_random(oracle, objective):
    rng = np.random.default_rng(5)
    n, F = 3000, 7
    X = rng.normal(size=(n, F)).astype(np.float32)
    X[rng.random((n, F)) < 0.05] = np.nan
    w = rng.normal(size=F)
    s = np.nan_to_num(X) @ w
    y = (s + 0.1 * rng.normal(size=n)).astype(np.float32) if objective == 0 else (s > 0).astype(np.float32)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 31, "double_precision": True},
           "tree": {"max_depth": 4, "eta": 0.3, "lambda": 1.0}}
    b = oracle.Booster(X, y=y, config=cfg)
    b.grow(1)
    leaf = b.leaf()
    bins = b.bins()
    tr = b.tree(0)
    # the leaf of every row equals a host traversal on its bins
    D = 5
    for i in range(0, n, 7):
        nd = 0
        for level in range(D - 1):
            idx = (1 << level) - 1 + nd
            q, f = tr["quantized"][idx], tr["fid"][idx]
            right = int(q >= 0 and bins[i, f] >= q + 1)
            nd = nd * 2 + right
        assert nd == leaf[i]
    # counts: sum over bins = node size; parent = left + right on the integers
    for level in range(D - 1):
        h = b.level_hist(level)
        tot = h[:, :, :, 2].sum(axis=2)
        assert np.all(tot == tot[:, :1])
        if level > 0:
            hp = b.level_hist(level - 1)
            assert np.array_equal(h[0::2] + h[1::2], hp)
    # with and without the subtraction trick: identical integers, identical tree
    cfg2 = dict(cfg, internals=dict(cfg["internals"], use_hist_subtraction_trick=False))
    b2 = oracle.Booster(X, y=y, config=cfg2)
    b2.grow(1)
    assert np.array_equal(b2.leaf(), leaf)
    for level in range(D - 1):
        assert np.array_equal(b.level_hist(level), b2.level_hist(level))
    # fixed-point sums against native double accumulation: 1e-5 relative
    b3 = oracle.Booster(X, y=y, config=cfg, accum=1)
    b3.grow(1)
    assert np.array_equal(b3.leaf(), leaf)
    for level in range(D - 1):
        a, c = b.level_hist(level, mode=1), b3.level_hist(level, mode=1)
        assert np.allclose(a, c, rtol=1e-5, atol=1e-6)
    # training-set prediction equals the tracked y_hat except where the raw-value
    # walk differs from the bin walk: a value exactly on a threshold, or a NaN
    # in an unsplit node (threshold +INF sends NaN right, training keeps it left)
    tracked = b.yhat() if objective == 0 else 1 / (1 + np.exp(-b.yhat().astype(np.float64)))
    clean = ~np.isnan(X).any(axis=1)
    assert np.allclose(b.predict(X)[clean], tracked[clean], atol=1e-5)


def test_baseline_config_0_on_the_oracle(oracle):
    # The CPU-runnable benchmark configuration: 10,000 x 28 ~ N(0,1), y = X.w + 0.1 N(0,1), squared
    # error, 256 bins, max_depth 6, eta 0.3, lambda 1, 10 trees.  The training error must fall with
    # every tree, and predicting the training rows must reproduce the kept y_hat.
    rng = np.random.default_rng(0)
    X = rng.standard_normal(size=(10000, 28), dtype=np.float32)
    w = rng.standard_normal(28)
    y = (X @ w + 0.1 * rng.standard_normal(10000)).astype(np.float32)
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 256, "double_precision": True},
           "tree": {"max_depth": 6, "eta": 0.3, "lambda": 1.0}}
    ob = oracle.Booster(X, y=y, config=cfg)
    errors = []
    for _ in range(10):
        ob.grow(1)
        errors.append(float(np.mean((ob.yhat() - y) ** 2)))
    assert all(b < a for a, b in zip(errors, errors[1:]))
    assert errors[-1] < 0.25 * np.var(y)
    assert np.allclose(ob.predict(X), ob.yhat(), atol=1e-5)


# ----------------------------------------------------------------- soft-max
# The reference's soft-max gradient kernel is empty; what it holds is the formula in the
# comment at src/core/objective.cu:60-89 (g = [k == label] - p_k, h = 2 p_k (1 - p_k)) and
# the link at src/core/objective.h:80-113.  The checks below pin the checker's restatement
# with routines that share no code with it: float64 numpy / scipy soft-max, the logistic
# special case, and what the mathematics fixes.
def _softmax_problem(K, n=4000, F=6, seed=11):
    rng = np.random.default_rng(seed)
    X = rng.normal(size=(n, F)).astype(np.float32)
    W = rng.normal(size=(F, K))
    labels = np.argmax(X @ W + rng.gumbel(size=(n, K)), axis=1).astype(np.uint8)
    return X, labels


def _softmax_cfg(K, objective=4, eta=0.5):
    return {"objective": objective, "method": 1, "internals": {"hist_size": 63, "double_precision": True},
            "tree": {"max_depth": 3, "eta": eta, "lambda": 1.0, "labels_count": K}}


@pytest.mark.parametrize("objective", [3, 4])
@pytest.mark.parametrize("K", [2, 3, 10])
def test_softmax_gradients_against_an_independent_softmax(oracle, objective, K):
    from scipy.special import softmax
    X, labels = _softmax_problem(K)
    b = oracle.Booster(X, labels=labels, config=_softmax_cfg(K, objective))
    n = X.shape[0]
    for rnd in range(3):
        raw = b.yhat().astype(np.float64).reshape(K, n)     # class-major scores before the round
        b.grow(1)
        g, h = (a.astype(np.float64).reshape(K, n) for a in b.grad())
        p = softmax(raw, axis=0)
        onehot = (np.arange(K)[:, None] == labels[None, :]).astype(np.float64)
        assert np.allclose(g, onehot - p, rtol=1e-6, atol=2e-7), "round %d" % rnd
        assert np.allclose(h, 2.0 * p * (1.0 - p), rtol=1e-6, atol=2e-7), "round %d" % rnd
        # what the mathematics fixes whatever the scores are
        assert np.all(np.abs(g.sum(axis=0)) < 1e-6 * K)      # probabilities sum to one
        assert h.min() >= 0.0 and h.max() <= 0.5             # 2 p (1 - p) on [0, 1]
        lab_g = g[labels, np.arange(n)]
        assert lab_g.min() >= 0.0                            # the label's own class is pushed up
        assert (g.sum(axis=0) - lab_g).max() <= 0.0          # every other class down
    # after the first round the scores differ between classes and rows
    assert np.ptp(raw, axis=0).max() > 0.1


def test_softmax_two_classes_is_the_logistic_sigmoid(oracle):
    # K = 2: p_1 = sigmoid(s_1 - s_0); g_1 = y - p_1 and h = 2 p_1 (1 - p_1), i.e. twice the
    # hessian of the (separately pinned) logistic objective on the score difference.
    X, labels = _softmax_problem(2, seed=3)
    b = oracle.Booster(X, labels=labels, config=_softmax_cfg(2))
    n = X.shape[0]
    b.grow(2)
    raw = b.yhat().reshape(2, n)
    b.grow(1)
    g, h = (a.reshape(2, n) for a in b.grad())
    d = (raw[1].astype(np.float64) - raw[0].astype(np.float64))
    s = np.array([oracle.lib().orc_sigmoid(float(v)) for v in d.astype(np.float32)], np.float64)
    assert np.allclose(g[1], labels - s, atol=3e-7)
    assert np.allclose(g[0], -(labels - s), atol=3e-7)
    assert np.allclose(h[1], 2 * s * (1 - s), atol=3e-7)
    assert np.allclose(h[0], h[1], atol=3e-7)


def test_softmax_link_against_scipy(oracle):
    from scipy.special import softmax
    K = 5
    X, labels = _softmax_problem(K, seed=7)
    b = oracle.Booster(X, labels=labels, config=_softmax_cfg(K))
    n = X.shape[0]
    b.grow(4)
    # rows without a value exactly on a threshold: prediction walks the raw floats to the same
    # leaves as training walked the bins, so the tracked scores are the raw scores of predict()
    raw = b.yhat().astype(np.float64).reshape(K, n).T        # row-major (n, K)
    out = b.predict(X)
    assert out.shape == (n, K)                               # objective.h:93-95: row-major out
    assert np.allclose(out.sum(axis=1), 1.0, atol=1e-6)
    assert np.allclose(out, softmax(raw, axis=1), rtol=1e-6, atol=1e-7)
    # n_rounds counts TREES (garden.cu:643-657): K trees = one round
    b1 = oracle.Booster(X, labels=labels, config=_softmax_cfg(K))
    b1.grow(1)
    assert np.array_equal(b.predict(X, n_rounds=K), b1.predict(X))
    # training moves probability mass towards the labels
    p0 = np.full(n, 1.0 / K)
    assert out[np.arange(n), labels].mean() > p0.mean() + 0.05


def test_softmax_gradient_is_the_derivative_of_the_log_likelihood(oracle):
    # g_k = d/ds_k log p_label by central differences on the checker's own link: ties the
    # gradient formula to the link function instead of to a second soft-max routine.
    from scipy.special import log_softmax
    K = 4
    X, labels = _softmax_problem(K, n=500, seed=5)
    b = oracle.Booster(X, labels=labels, config=_softmax_cfg(K))
    n = X.shape[0]
    b.grow(2)
    raw = b.yhat().astype(np.float64).reshape(K, n)
    b.grow(1)
    g = b.grad()[0].astype(np.float64).reshape(K, n)
    eps = 1e-5
    for k in range(K):
        up, dn = raw.copy(), raw.copy()
        up[k] += eps
        dn[k] -= eps
        num = (log_softmax(up, axis=0)[labels, np.arange(n)] - log_softmax(dn, axis=0)[labels, np.arange(n)]) / (2 * eps)
        assert np.allclose(g[k], num, atol=1e-6)


def test_heavy_tailed_regression_fixed_point_keeps_the_split_choice(oracle):
    # Squared error scales the fixed point by the round's largest residual: with five targets
    # 2^21 times larger than the rest a typical residual keeps 7 fractional bits.  The splits
    # must still be those of fp64 accumulation (the reference's double_precision=true sums).
    rng = np.random.default_rng(1)
    n, F = 20000, 8
    X = rng.normal(size=(n, F)).astype(np.float32)
    y = (X[:, 0] * 2 + np.sin(X[:, 1] * 3) + 0.1 * rng.normal(size=n)).astype(np.float32)
    y[rng.choice(n, 5, replace=False)] *= 2.0 ** 21
    cfg = {"objective": 0, "method": 1, "internals": {"hist_size": 63, "double_precision": True},
           "tree": {"max_depth": 5, "eta": 0.3, "lambda": 1.0, "min_leaf_size": 50}}
    fixed, native = oracle.Booster(X, y=y, config=cfg, accum=0), oracle.Booster(X, y=y, config=cfg, accum=1)
    for r in range(4):
        fixed.grow(1)
        native.grow(1)
        a, b = fixed.tree(r), native.tree(r)
        assert fixed.shifts()[0] <= 8
        assert np.array_equal(a["fid"], b["fid"]) and np.array_equal(a["quantized"], b["quantized"])
        # nodes that hold no outlier see the coarse scale: their gains agree to 1e-3 relative only
        # (the documented limit of one scale per round), nodes with outliers to 1e-5
        assert np.allclose(a["gain"], b["gain"], rtol=2e-3)
        big = b["gain"] > 1e6
        assert big.any() and np.allclose(a["gain"][big], b["gain"][big], rtol=1e-5)
        assert np.allclose(a["weights"], b["weights"], rtol=1e-5, atol=1e-3)
    assert np.array_equal(fixed.leaf(), native.leaf())


def test_logistic_labels_outside_0_1_keep_their_gradients(oracle):
    # the fixed-point scale follows the label range: no row's gradient is dropped
    rng = np.random.default_rng(2)
    X = rng.normal(size=(3000, 4)).astype(np.float32)
    y = np.where(X[:, 0] > 0, 1.0, -1.0).astype(np.float32)
    cfg = {"objective": 1, "method": 1, "internals": {"hist_size": 31, "double_precision": True},
           "tree": {"max_depth": 3, "eta": 0.3, "lambda": 1.0}}
    b = oracle.Booster(X, y=y, config=cfg)
    b.grow(1)
    assert b.shifts() == (28, 32)
    g, _ = b.grad()
    assert g.min() < -1.0      # y = -1 rows: g = -1 - s
    root = b.level_hist(0)[0, 0]
    assert int(root[:, 0].sum()) == int(np.rint(g.astype(np.float64) * 2.0 ** 28).sum())
    native = oracle.Booster(X, y=y, config=cfg, accum=1)
    native.grow(1)
    assert np.array_equal(b.tree(0)["fid"], native.tree(0)["fid"])
    assert np.array_equal(b.tree(0)["quantized"], native.tree(0)["quantized"])


# ------------------------------------------------------- column sampling
# Reference: InitGrowingTree / InitTreeLevel / FindBestSplits, src/core/garden.cu:126-165, 249-253.
# The literal id vectors of column_sampling.json come from tests/golden/make_shuffle_vectors.cpp,
# which holds the reference's calls on its random engine and nothing else.
def _sampling_booster(oracle, case, trees, max_depth, objective=1, rows=600):
    rng = np.random.default_rng(17)
    F = case["columns"]
    X = rng.normal(size=(rows, F)).astype(np.float32)
    s = X @ rng.normal(size=F)
    y = (s > 0).astype(np.float32) if objective else (s + 0.1 * rng.normal(size=rows)).astype(np.float32)
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": 16, "double_precision": True, "seed": case["seed"]},
           "tree": {"max_depth": max_depth, "eta": 0.3, "lambda": 1.0, "min_child_weight": 0.0,
                    "colsample_bytree": case["colsample_bytree"], "colsample_bylevel": case["colsample_bylevel"]}}
    b = oracle.Booster(X, y=y, config=cfg, accum=1)
    b.grow(trees)
    return b, X, y, cfg


@pytest.mark.parametrize("case", load_golden("column_sampling.json"),
                         ids=lambda c: "seed%d-F%d-%g-%g" % (c["seed"], c["columns"], c["colsample_bytree"],
                                                             c["colsample_bylevel"]))
def test_column_sampling_active_ids_equal_the_reference_call_sequence(oracle, case):
    # A re-shuffle of the wrong range (all ids instead of the first int(bytree*F)), a wrong prefix
    # (bytree*F instead of bylevel*bytree*F ids), ids not reset per tree, or one engine per tree
    # instead of one per booster all change these vectors.
    trees, levels = len(case["active"]), len(case["active"][0])
    b, _, _, _ = _sampling_booster(oracle, case, trees, levels)
    F, bt, bl = case["columns"], np.float32(case["colsample_bytree"]), np.float32(case["colsample_bylevel"])
    per_tree, per_level = int(bt * np.float32(F)), int(np.float32(bl * bt) * np.float32(F))
    for t in range(trees):
        seen = set()
        for level in range(levels):
            ids = b.active_features(t, level).tolist()
            assert ids == case["active"][t][level], (t, level)
            assert len(ids) == per_level and len(set(ids)) == per_level
            seen |= set(ids)
            # every split of the level uses one of its active features
            tr = b.tree(t)
            for nd in range((1 << level) - 1, (2 << level) - 1):
                if tr["quantized"][nd] >= 0:
                    assert tr["fid"][nd] in ids, (t, level, nd)
        assert len(seen) <= per_tree       # the levels draw from the tree's int(bytree*F) ids only
    with pytest.raises(IndexError):
        b.active_features(trees, 0)


def test_column_sampling_fixture_tells_the_shuffle_ranges_apart():
    # the fixture must be able to fail: with bytree < 1 some level of some tree shows an id set
    # that differs from the previous level's (the per-level re-shuffle is visible), and the
    # trees differ from each other (one engine per booster, ids reset per tree)
    for case in load_golden("column_sampling.json"):
        if case["colsample_bytree"] * case["colsample_bylevel"] == 1.0:
            assert all(sorted(lv) == list(range(case["columns"])) for tr in case["active"] for lv in tr)
            continue
        assert any(tr[i] != tr[i + 1] for tr in case["active"] for i in range(len(tr) - 1))
        assert case["active"][0] != case["active"][1]


@pytest.mark.parametrize("objective", [0, 1])
def test_column_sampling_searches_exactly_the_active_features(oracle, objective):
    # node by node: the split of a node is the brute-force best over the ACTIVE features of its
    # level (lowest feature id on equal gains, whatever the shuffled order), found on its own rows
    case = {"seed": 9, "columns": 6, "colsample_bytree": 0.7, "colsample_bylevel": 0.8}
    depth, lam = 3, 1.0
    b, X, y, cfg = _sampling_booster(oracle, case, 2, depth, objective=objective, rows=150)
    bins = b.bins().astype(np.float32)
    g, h = b.grad()                      # gradients of the LAST round = those tree 1 was grown on
    if objective == 0:
        h = np.ones_like(g)
    t = b.tree(1)
    rows = {0: np.arange(len(y))}
    some_feature_left_out = False
    for i in range((1 << depth) - 1):
        level = int(np.log2(i + 1))
        act = np.sort(b.active_features(1, level))
        assert len(act) == int(np.float32(np.float32(0.7) * np.float32(0.8)) * np.float32(6)) == 3
        r = rows[i]
        f = -1
        if len(r) > 1:
            f, first_right, gain = _brute_force_exact_root(oracle, bins[np.ix_(r, act)], g[r], h[r],
                                                           1 if objective == 0 else 3, (1, 0.0, 0.0, 0.0, lam, 0.0))
            all_f, _, all_gain = _brute_force_exact_root(oracle, bins[r], g[r], h[r],
                                                         1 if objective == 0 else 3, (1, 0.0, 0.0, 0.0, lam, 0.0))
            some_feature_left_out |= all_f >= 0 and all_f not in act and (f < 0 or all_gain > gain)
        if f >= 0:
            assert (t["fid"][i], t["quantized"][i]) == (act[f], int(first_right) - 1), "node %d" % i
            assert t["gain"][i] == pytest.approx(gain, rel=1e-5)
            right = bins[r, act[f]] >= first_right
        else:
            assert t["quantized"][i] == -1 and t["fid"][i] == 0, "node %d" % i
            right = np.zeros(len(r), bool)
        rows[2 * i + 1], rows[2 * i + 2] = r[~right], r[right]
    assert some_feature_left_out         # sampling changed at least one decision on this input


def test_column_sampling_same_seed_same_trees_and_ratio_one_is_no_sampling(oracle):
    case = {"seed": 4, "columns": 9, "colsample_bytree": 0.6, "colsample_bylevel": 0.9}
    a, X, y, cfg = _sampling_booster(oracle, case, 3, 3)
    b, _, _, _ = _sampling_booster(oracle, case, 3, 3)
    c, _, _, _ = _sampling_booster(oracle, dict(case, seed=5), 3, 3)
    same = lambda p, q: all(np.array_equal(p.tree(t)[k], q.tree(t)[k]) for t in range(3)
                            for k in ("fid", "quantized", "weights"))
    assert same(a, b) and not same(a, c)
    full = dict(case, colsample_bytree=1.0, colsample_bylevel=1.0)
    d, _, _, _ = _sampling_booster(oracle, full, 3, 3)
    e, _, _, _ = _sampling_booster(oracle, dict(full, seed=77), 3, 3)       # the order drawn does not matter
    assert same(d, e) and not same(a, d)
    assert sorted(d.active_features(2, 1).tolist()) == list(range(9))


def test_column_sampling_too_small_raises_the_reference_messages(oracle):
    # garden.cu:127-140: the two literals, the first one wins; nothing is grown
    X = np.random.default_rng(0).normal(size=(50, 3)).astype(np.float32)
    y = (X[:, 0] > 0).astype(np.float32)
    for tree, msg in (({"colsample_bytree": 0.1}, "colsample_bytree is too small"),
                      ({"colsample_bytree": 0.1, "colsample_bylevel": 0.1}, "colsample_bytree is too small"),
                      ({"colsample_bytree": 0.5, "colsample_bylevel": 0.5},
                       "colsample_bytree and colsample_bylevel are too small")):
        b = oracle.Booster(X, y=y, config={"objective": 1, "method": 1, "tree": dict(tree, max_depth=2)})
        with pytest.raises(ValueError) as e:
            b.grow(1)
        assert str(e.value) == msg and b.num_trees == 0
