"""CPU-side tests of the C-ABI library: it loads without a GPU, exports every
symbol the headers declare, and its host-only entry points (configuration,
model JSON, prediction) behave like the reference's."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "arboretum_amd", "libarboretum.so")


def declared_symbols():
    names = []
    for header in ("arboretum_wrapper.h", "arboretum_ext.h"):
        text = open(os.path.join(ROOT, "include", header)).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        names += re.findall(r"const char \*(A\w+)\(", text)
    return names


def test_library_exports_every_declared_symbol():
    assert os.path.exists(LIB), "libarboretum.so is not built (python arboretum_amd/build.py)"
    lib = ctypes.CDLL(LIB)
    names = declared_symbols()
    # the 14 entry points of python-wrapper/arboretum_wrapper.h:6-39
    for ref in ["ACreateFromDenseMatrix", "ASetY", "ASetLabel", "ASetWeights", "AInitGarden", "AGrowTree",
                "AAppendLastTree", "AGetY", "APredict", "ADumpModel", "ALoadModel", "AFreeDMatrix",
                "AFreeGarden", "ADeleteArray"]:
        assert ref in names
    for n in names:
        assert hasattr(lib, n), n


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    return arboretum_amd


def test_import_alias(arb):
    import arboretum
    assert arboretum.DMatrix is arb.DMatrix and arboretum.Garden is arb.Garden


def test_configuration_round_trip(arb):
    cfg = {"objective": 1, "method": 1,
           "internals": {"double_precision": True, "compute_overlap": 3, "hist_size": 12, "seed": 7,
                         "use_hist_subtraction_trick": False, "upload_features": False},
           "tree": {"eta": 0.99999, "max_depth": 3, "gamma": 0.0, "min_child_weight": 2, "min_leaf_size": 2,
                    "lambda": 0.0, "alpha": 0.5, "max_leaf_weight": 1.5, "gamma_absolute": 0.25},
           "verbose": {"gpu": True}}
    g = arb.Garden(cfg)
    conf = json.loads(g.dump())["configuration"]
    # float32 values print as the shortest double that round-trips (json_conversion.h / nlohmann)
    assert conf["tree"]["eta"] == 0.9999899864196777
    assert conf["tree"]["max_depth"] == 3 and conf["tree"]["min_leaf_size"] == 2
    assert conf["tree"]["min_child_weight"] == 2.0 and conf["tree"]["alpha"] == 0.5
    assert conf["tree"]["lambda"] == 0.0 and conf["tree"]["initial_y"] == 0.5 and conf["tree"]["labels_count"] == 1
    assert conf["internals"] == {"compute_overlap": 3, "double_precision": True, "hist_size": 12, "seed": 7,
                                 "upload_features": False, "use_hist_subtraction_trick": False}
    assert conf["verbose"] == {"booster": False, "data": False, "gpu": True}
    assert conf["method"] == 1 and conf["objective"] == 1
    assert json.loads(g.dump())["model"] == []


def test_defaults_follow_reference(arb):
    conf = json.loads(arb.Garden({"objective": 0, "method": 1}).dump())["configuration"]
    t, it = conf["tree"], conf["internals"]      # src/core/param.h:21-27,54-57
    assert t["max_depth"] == 7 and t["min_child_weight"] == 1.0 and t["min_leaf_size"] == 1
    assert t["lambda"] == 1.0 and t["alpha"] == 0.0 and t["initial_y"] == 0.5
    assert abs(t["eta"] - 0.3) < 1e-7 and t["colsample_bytree"] == 1.0
    assert it["hist_size"] == 255 and it["use_hist_subtraction_trick"] and it["upload_features"]
    assert it["compute_overlap"] == 2 and it["seed"] == 0 and not it["double_precision"]


@pytest.mark.parametrize("bad", ["{", "[1,2]", '{"tree": {"max_depth": "x"}}', '{"objective": 7}',
                                 '{"tree": {"max_depth": 0}}', '{"tree": {"max_depth": 40}}'])
def test_bad_configuration_is_an_error_string(arb, bad):
    lib = ctypes.CDLL(LIB)
    lib.AInitGarden.restype = ctypes.c_char_p
    h = ctypes.c_void_p()
    msg = lib.AInitGarden(bad.encode(), ctypes.byref(h))
    assert msg is not None and len(msg) > 0


def _golden(name):
    with open(os.path.join(ROOT, "tests", "golden", name)) as f:
        return json.load(f)


def test_load_golden_model_and_predict_on_host(arb):
    # model JSON of tests/py/test_hist_regregression.py; prediction is host code
    fx = _golden("hist_regression_boston10.json")
    X = np.array(fx["X"], np.float32)
    data = arb.DMatrix(X, y=np.array(fx["y"], np.float32))
    for name, case in fx["cases"].items():
        true = case["true_model"]
        for tree in true["model"]:
            tree.setdefault("depth", case["max_depth"] + 1)   # the goldens predate the "depth" key
        model = arb.load(json.dumps(true))
        for i in range(case["trees"]):
            assert np.allclose(model.predict(data, i + 1), case["true_values"][i]), name
        again = json.loads(model.dump())
        for tt, ct in zip(true["model"], again["model"]):
            assert tt["nodes"] == ct["nodes"]
            assert np.allclose(tt["weights"], ct["weights"], rtol=1e-6)
        # n_rounds counts trees; 0 trees gives the initial value
        assert np.allclose(model.predict(data, 0), 0.5)


def test_load_golden_logistic_model(arb):
    fx = _golden("hist_logistic_iris.json")
    X = np.array(fx["X"], np.float32)
    data = arb.DMatrix(X, y=(np.array(fx["target"]) != 2).astype(np.float32))
    for name, case in fx["cases"].items():
        true = case["true_model"]
        for tree in true["model"]:
            tree.setdefault("depth", case["max_depth"] + 1)
        model = arb.load(json.dumps(true))
        for i in range(case["trees"]):
            assert np.allclose(model.predict(data, i + 1), case["true_values"][i]), name


def test_append_last_tree_and_get_y(arb):
    fx = _golden("hist_regression_boston10.json")
    case = fx["cases"]["test_2trees_depth_2"]
    true = case["true_model"]
    for tree in true["model"]:
        tree.setdefault("depth", 3)
    model = arb.load(json.dumps(true))
    ev = arb.DMatrix(np.array(fx["X"], np.float32))
    model.append_last_tree(ev)       # adds the LAST tree to y_hat (starts from initial_y)
    want = model.predict(ev, 2) - model.predict(ev, 1) + 0.5
    assert np.allclose(model.get_y(ev), want, atol=1e-5)


def test_null_threshold_loads_as_infinity(arb):
    model = {"configuration": {"objective": 0, "method": 1, "tree": {"max_depth": 1}},
             "model": [{"depth": 2, "weights": [1.5, -2.5],
                        "nodes": [{"id": 0, "leaf": False, "left": 1, "right": 2, "threshold": None, "fid": 0},
                                  {"id": 1, "leaf": True, "idx": 0}, {"id": 2, "leaf": True, "idx": 1}]}]}
    g = arb.load(json.dumps(model))
    X = np.array([[1.0], [np.nan], [np.inf]], np.float32)
    # x < +INF is left; NaN and +INF go right (garden.h:79-86)
    assert g.predict(arb.DMatrix(X)).tolist() == [2.0, -2.0, -2.0]
    assert json.loads(g.dump())["model"][0]["nodes"][0]["threshold"] is None


def test_training_without_gpu_fails_loudly(arb):
    if arb.device_count() > 0:
        pytest.skip("a GPU is present")
    X = np.random.default_rng(0).normal(size=(20, 3)).astype(np.float32)
    g = arb.Garden({"objective": 0, "method": 1, "tree": {"max_depth": 2}}, arb.DMatrix(X, y=X[:, 0]))
    with pytest.raises(arb.ArboretumError, match="no HIP device"):
        g.grow_tree()


@pytest.mark.parametrize("bad", [np.nan, np.inf, -np.inf])
@pytest.mark.parametrize("objective", [0, 1])
def test_non_finite_targets_are_refused(arb, bad, objective):
    # the fixed-point scale of the gradients has no meaning with a NaN or infinite target;
    # refused on the host, before any device work
    X = np.random.default_rng(0).normal(size=(50, 3)).astype(np.float32)
    y = (X[:, 0] > 0).astype(np.float32)
    y[17] = bad
    g = arb.Garden({"objective": objective, "method": 1, "tree": {"max_depth": 2}}, arb.DMatrix(X, y=y))
    with pytest.raises(arb.ArboretumError, match="y must be finite"):
        g.grow_tree()


def test_errors(arb):
    X = np.zeros((4, 2), np.float32)
    with pytest.raises(ValueError):
        arb.DMatrix(X, y=np.zeros(4), labels=np.zeros(4, np.uint8))
    with pytest.raises(ValueError):
        arb.DMatrix(np.zeros(4, np.float32))
    g = arb.Garden({"objective": 0, "method": 1})
    with pytest.raises(arb.ArboretumError):
        g.load('{"no_model": 1}')


def test_no_alloc_histogram_size_limits_are_checked_before_the_gpu_is_touched():
    # AHistSumNoAlloc keeps plan and slabs in a static device array (32 MB of slabs, at most
    # 1024 work items of at most 64512 rows, two spare items per node): what cannot fit is
    # refused on the host.  The addresses below are never dereferenced by host code.
    import arboretum_amd as arb
    p = 4096

    def refused(stride, nrow, ncol, nodes):
        try:
            arb.hist_sum_no_alloc(p, p, p, p, p, p, p, stride, nrow, ncol, nodes, 30, 32)
        except arb.ArboretumError as e:
            return "too large for the static work memory" in str(e)
        return False
    assert refused(20000000, 20000000, 28, 1)            # 256 items x 64512 rows < 20 M rows
    assert refused(64512 * 200, 64512 * 200, 28, 64)     # 128 of the 256 items go to the 64 nodes
    assert refused(1024, 1000, 600, 6)                   # 2.4 MB per slab: 13 items < 2 * 6 + 2
    assert refused(1 << 20, 1 << 20, 2100, 1)            # 8.4 MB per slab: 3 items
    # sizes that fit pass the size check (and then fail here only for want of a GPU)
    if arb.device_count() == 0:
        with pytest.raises(arb.ArboretumError, match="HIP error"):
            arb.hist_sum_no_alloc(p, p, p, p, p, p, p, 8000000, 8000000, 28, 64, 30, 32)
    with pytest.raises(arb.ArboretumError, match="sibling pairs"):
        arb.hist_sum_no_alloc(p, p, p, p, p, p, p, 1024, 1000, 28, 3, 30, 32, use_trick=True, parent_g=p,
                              parent_h=p, parent_c=p)


def test_hist_sum_plans_items_of_the_largest_size_for_many_rows(arb):
    # about 512 work items while items of at most 64512 rows allow it; beyond 512 x 64512 = 33 M rows
    # the items keep that size and their number grows (it must not fall back to 1024-row items:
    # 50 M rows would then take 49 000 slabs of 128 KB)
    per, items = arb.hist_sum_plan(10_500_000, 1)
    assert per % 1024 == 0 and 500 <= items <= 520 and per * (items - 4) <= 10_500_000 <= per * items
    for rows, nodes in ((33_100_000, 1), (50_000_000, 8), (2_000_000_000, 64)):
        per, items = arb.hist_sum_plan(rows, nodes)
        assert per == 64512, (rows, per)
        assert items == rows // 64512 + 2 * nodes + 2
    per, items = arb.hist_sum_plan(1000, 2)
    assert per == 1024 and items == 6


def test_block_matrix_arguments_are_checked_on_the_host(arb):
    # ACreateFromQuantizedBlocks: nothing is dereferenced when the matrix is created
    p, br = 4096, 1 << 30
    for blocks, block_rows, rows, msg in (([p], 100, 100, "multiple of 64"),
                                          ([p], 1 << 31, 1 << 31, "fewer than 2\\^31"),
                                          ([p, p], 128, 128, "does not match"),
                                          ([p, 0], 128, 200, "null block"),
                                          # integer gradient sums of 2^30 per row leave 64 bits from 2^33 rows on
                                          ([p] * 8, br, 1 << 33, "fewer than 2\\^33 rows")):
        with pytest.raises(arb.ArboretumError, match=msg):
            arb.DMatrix.from_blocks(blocks, block_rows, rows, 4)


def test_tree_arrays_follow_the_depth_of_a_loaded_tree(arb):
    # a model whose trees are deeper (and shallower) than the booster's configuration
    def tree(depth):
        ni = (1 << (depth - 1)) - 1
        nodes = [{"id": i, "leaf": False, "left": 2 * i + 1, "right": 2 * i + 2, "threshold": float(i), "fid": i % 3}
                 for i in range(ni)]
        nodes += [{"id": ni + k, "leaf": True, "idx": k} for k in range(1 << (depth - 1))]
        return {"nodes": nodes, "weights": [float(k) for k in range(1 << (depth - 1))], "depth": depth}
    g = arb.Garden({"objective": 0, "method": 1, "tree": {"max_depth": 2}})
    g.load(json.dumps({"model": [tree(5), tree(2)]}))
    deep, shallow = g.tree(0), g.tree(1)
    assert deep["fid"].shape == (15,) and deep["weights"].shape == (16,)
    assert shallow["fid"].shape == (1,) and shallow["weights"].tolist() == [0.0, 1.0]
    assert deep["weights"].tolist() == [float(k) for k in range(16)]
    assert deep["threshold"].tolist() == [float(i) for i in range(15)]
