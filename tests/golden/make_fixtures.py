"""Writes the golden fixtures under tests/golden/ (data only).

The reference's pytest files are parsed as TEXT with `ast` (nothing from the
reference is imported or executed): for every hist-method test the literal
arguments of its `run_regression(depth, true_values, json.loads('<model>'),
trees)` call are copied into a JSON fixture, together with the data set the
test trains on (Boston rows 0..9, Iris) taken from the CSV files that ship
with scikit-learn.  The quantiser / histogram / gain vectors of the
reference's C++ tests are small enough to be written out here by the formulas
those tests state (file:line given per case).

Run once in the build container:  python tests/golden/make_fixtures.py
"""
import ast
import csv
import json
import os
import sys

REF = os.environ.get("ARBORETUM_REFERENCE", "/root/reference")
HERE = os.path.dirname(os.path.abspath(__file__))


def _calls(path):
    tree = ast.parse(open(path).read())
    out = {}
    for fn in tree.body:
        if not isinstance(fn, ast.FunctionDef) or not fn.name.startswith("test_"):
            continue
        for node in ast.walk(fn):
            if isinstance(node, ast.Call) and getattr(node.func, "id", "") == "run_regression":
                depth = ast.literal_eval(node.args[0])
                values = ast.literal_eval(node.args[1])
                model = json.loads(ast.literal_eval(node.args[2].args[0]))
                trees = ast.literal_eval(node.args[3]) if len(node.args) > 3 else 1
                out[fn.name] = {"max_depth": depth, "trees": trees, "true_values": values,
                                "true_model": model}
    return out


def _config_of(path):
    """The literal `config = {...}` dict of run_regression, names left as strings."""
    tree = ast.parse(open(path).read())
    for fn in tree.body:
        if isinstance(fn, ast.FunctionDef) and fn.name == "run_regression":
            for node in ast.walk(fn):
                if isinstance(node, ast.Assign) and getattr(node.targets[0], "id", "") == "config":
                    def ev(n):
                        if isinstance(n, ast.Dict):
                            return {ev(k): ev(v) for k, v in zip(n.keys, n.values)}
                        if isinstance(n, ast.Name):
                            return "$" + n.id
                        return ast.literal_eval(n)
                    return ev(node.value)
    raise RuntimeError("config not found in " + path)


def boston10():
    import sklearn
    p = os.path.join(os.path.dirname(sklearn.__file__), "datasets", "data", "boston_house_prices.csv")
    if not os.path.exists(p):
        p = "/opt/conda/lib/python3.9/site-packages/sklearn/datasets/data/boston_house_prices.csv"
    rows = list(csv.reader(open(p)))[2:12]
    X = [[float(v) for v in r[:13]] for r in rows]
    y = [float(r[13]) for r in rows]
    return X, y


def iris():
    import sklearn
    p = os.path.join(os.path.dirname(sklearn.__file__), "datasets", "data", "iris.csv")
    rows = list(csv.reader(open(p)))[1:]
    X = [[float(v) for v in r[:4]] for r in rows]
    t = [int(r[4]) for r in rows]
    return X, t


def main():
    reg = os.path.join(REF, "tests/py/test_hist_regregression.py")
    log = os.path.join(REF, "tests/py/test_hist_logregression.py")
    X, y = boston10()
    json.dump({"source": "tests/py/test_hist_regregression.py:13-56 (config), :58-138 (cases)",
               "X": X, "y": y, "config": _config_of(reg), "cases": _calls(reg)},
              open(os.path.join(HERE, "hist_regression_boston10.json"), "w"))
    X, t = iris()
    json.dump({"source": "tests/py/test_hist_logregression.py:9-66 (config), :69-162 (cases)",
               "X": X, "target": t, "config": _config_of(log), "cases": _calls(log)},
              open(os.path.join(HERE, "hist_logistic_iris.json"), "w"))

    # ---- exact-method goldens (method 0), tests/py/test_regression.py and test_logresression.py
    ereg = os.path.join(REF, "tests/py/test_regression.py")
    elog = os.path.join(REF, "tests/py/test_logresression.py")
    X, y = boston10()
    json.dump({"source": "tests/py/test_regression.py:14-53 (config), :56-91 (cases)",
               "X": X, "y": y, "config": _config_of(ereg), "cases": _calls(ereg)},
              open(os.path.join(HERE, "exact_regression_boston10.json"), "w"))
    X, t = iris()
    json.dump({"source": "tests/py/test_logresression.py:9-43 (config), :46-135 (cases)",
               "X": X, "target": t, "config": _config_of(elog), "cases": _calls(elog)},
              open(os.path.join(HERE, "exact_logistic_iris.json"), "w"))

    # ---- sklearn-style classifier golden, tests/py/test_sklearn_classification.py:9-61: the default
    # value of the test's `y_pred` argument and the keyword arguments of its ArboretumClassifier(...)
    cls = os.path.join(REF, "tests/py/test_sklearn_classification.py")
    tree = ast.parse(open(cls).read())
    fn = next(f for f in tree.body if isinstance(f, ast.FunctionDef) and f.name == "test_single_tree")
    y_pred = ast.literal_eval(fn.args.defaults[-1])[0]
    call = next(n for n in ast.walk(fn) if isinstance(n, ast.Call) and getattr(n.func, "attr", "") == "ArboretumClassifier")
    params = {}
    for kw in call.keywords:
        params[kw.arg] = "$" + kw.value.id if isinstance(kw.value, ast.Name) else ast.literal_eval(kw.value)
    sweep = {}
    for dec in fn.decorator_list:  # @pytest.mark.parametrize("name", [values])
        sweep[ast.literal_eval(dec.args[0])] = ast.literal_eval(dec.args[1])
    Xi, ti = iris()
    json.dump({"source": "tests/py/test_sklearn_classification.py:9-61", "X": Xi, "target": ti,
               "label_rule": "target != 2", "params": params, "sweep": sweep, "y_pred": y_pred},
              open(os.path.join(HERE, "sklearn_classification_iris.json"), "w"))

    # ---- quantiser goldens, tests/cpp/test_datamatrix.cu
    q = []
    q.append({"name": "HistWideRange", "cite": "tests/cpp/test_datamatrix.cu:25-46", "hist_size": 8,
              "x": [float(128 - i) for i in range(128)],
              "bins": [8 - (i // 16) - 1 for i in range(128)], "bits": 4})
    q.append({"name": "Hist255", "cite": "tests/cpp/test_datamatrix.cu:48-72", "hist_size": 255,
              "x": [float(i) for i in range(1024)],
              "bins": [(i // 4) if i < 1020 else 254 for i in range(1024)], "bits": 8})
    q.append({"name": "HistSkewedRange", "cite": "tests/cpp/test_datamatrix.cu:74-112", "hist_size": 4,
              "x": [10, 0, 11, 1, 0, 2, 3, 0, 0, 0, 0, 0], "bins": [3, 0, 3, 1, 0, 2, 3, 0, 0, 0, 0, 0],
              "bits": 3})
    q.append({"name": "HistTinyRange1", "cite": "tests/cpp/test_datamatrix.cu:114-152", "hist_size": 4,
              "x": [0, 0, 0, 1, 0, 2, 0, 0, 0, 0, 0, 0], "bins": [0, 0, 0, 1, 0, 2, 0, 0, 0, 0, 0, 0],
              "bits": 2})
    q.append({"name": "HistTinyRange2", "cite": "tests/cpp/test_datamatrix.cu:154-197", "hist_size": 4,
              "x": [10, 10, 10, 1, 10, 2, 10, 10, 10, 10, 10, 10], "bins": [0] * 12, "bits": 1,
              "first_threshold_inf": True})
    json.dump(q, open(os.path.join(HERE, "quantiser.json"), "w"))

    # ---- gain / arg-max goldens, tests/cpp/test_hist.cu
    g = []
    # :80-121 root: 32 rows, grad (i,1), bin i/8, hist 4 -> idx 1, gain 2048
    g.append({"name": "RootSearch", "cite": "tests/cpp/test_hist.cu:80-121", "hist_size": 4,
              "params": [0, 0, 0, 0, 0, 0], "nodes": [
                  {"bins": [i // 8 for i in range(32)], "g": [float(i) for i in range(32)],
                   "h": [1.0] * 32, "best_bin": 1, "gain": 2048.0}]})
    # :123-259 level 1: node 0 = positions 0..15 (bin p/2), node 1 = positions
    # 16..31 (bin 7-(p-16)/2), grad (p*p,1): best global idx 4 and 11
    # the same sums, best bins and gains are asserted by every Level1Search variant of the file
    # (NoTrickDynamic :123, _Upload :262, NoTrickStatic :594, WithTrickDynamic :702, WithTrickStatic
    # :811): they differ in how the reference gets there (launch mode, streaming, subtraction)
    g.append({"name": "Level1Search", "cite": "tests/cpp/test_hist.cu:123-259",
              "same_numbers_in": ["tests/cpp/test_hist.cu:262-400", "tests/cpp/test_hist.cu:594-700",
                                  "tests/cpp/test_hist.cu:702-809", "tests/cpp/test_hist.cu:811-921"],
              "hist_size": 8,
              "params": [0, 0, 0, 0, 0, 0], "nodes": [
                  {"bins": [p // 2 for p in range(16)], "g": [float(p * p) for p in range(16)],
                   "h": [1.0] * 16, "best_bin": 4, "gain": 64026.672,
                   "sums": [1, 13, 41, 85, 145, 221, 313, 421]},
                  {"bins": [7 - (p - 16) // 2 for p in range(16, 32)],
                   "g": [float(p * p) for p in range(16, 32)], "h": [1.0] * 16, "best_bin": 3,
                   "gain": 565504.0, "sums": [1861, 1625, 1405, 1201, 1013, 841, 685, 545]}]})
    json.dump(g, open(os.path.join(HERE, "gain.json"), "w"))

    # ---- histogram goldens: all 17 cases of tests/cpp/test_hist_sum.cu.  Every case has
    # grad[i] = float(i); "bins" names the rule of the test ("i", "0", "i%H"); "count" / "sum"
    # map the flat cell index node * H + bin to the value the test asserts, "node_sum" holds
    # the asserted totals over a node's cells.  The (BIN_T, SUM_T) variants of a test share
    # one set of numbers and differ in "bin_type" / "sum_type".
    h = []
    blk = 128  # HIST_SUM_BLOCK_DIM, src/core/hist_grad_sum.cuh:6
    variants = [("Float", "Bin16", 11, 71, 133), ("Float", "Bin8", 41, 102, 165),
                ("Double", "Bin16", 197, 257, 319), ("Double", "Bin8", 227, 288, 351)]
    for st, bt, l_naive, l_seg, l_full in variants:
        base = {"sum_type": st.lower(), "bin_type": bt.lower(), "trick": False, "parent_count": None,
                "parent_sum": None, "node_sum": None}
        h.append(dict(base, name="SingleNodeHistSum%s%s.Naive" % (st, bt),
                      cite="tests/cpp/test_hist_sum.cu:%d-%d" % (l_naive, l_naive + 28), rows=32, bins="i",
                      hist_size=32, node_size=[0, 32], count={str(i): 1 for i in range(32)},
                      sum={str(i): float(i) for i in range(32)}))
        h.append(dict(base, name="SingleNodeHistSum%s%s.SingleSegment" % (st, bt),
                      cite="tests/cpp/test_hist_sum.cu:%d-%d" % (l_seg, l_seg + 29), rows=32, bins="0",
                      hist_size=32, node_size=[0, 32], count={"0": 32}, sum={"0": float(32 * 31 // 2)}))
        n = blk * 10
        h.append(dict(base, name="SingleNodeHistSum%s%s.SingleSegmentFullSize" % (st, bt),
                      cite="tests/cpp/test_hist_sum.cu:%d-%d" % (l_full, l_full + 30), rows=n, bins="0",
                      hist_size=256, node_size=[0, n], count={"0": n}, sum={"0": float(n * (n - 1) // 2)}))
    n = blk * 10
    multi = {"sum_type": "double", "bin_type": "bin16", "rows": n, "hist_size": 4}
    h.append(dict(multi, name="MultiNodeHistSumDouble._2_NodesNoTrick", cite="tests/cpp/test_hist_sum.cu:383-424",
                  bins="i%H", node_size=[0, n // 2, n], trick=False, parent_count=None, parent_sum=None,
                  count={str(i): n // 8 for i in range(8)}, sum={},
                  node_sum=[float((n // 2) * (n // 2 - 1) // 2), float((n // 2) * (n // 2 + n - 1) // 2)]))
    asym_c = {str(i): v for i, v in enumerate([3, 3, 2, 2, 317, 317, 318, 318])}
    asym_s = {str(i): v for i, v in enumerate([12.0, 15.0, 8.0, 10.0, 204148.0, 204465.0, 204792.0, 205110.0])}
    par_c = [320, 320, 320, 320]
    par_s = [204148.0 + 12.0, 204465.0 + 15.0, 204792.0 + 8.0, 205110.0 + 10.0]
    h.append(dict(multi, name="MultiNodeHistSumDouble._2_NodesAsymmetricNoTrick",
                  cite="tests/cpp/test_hist_sum.cu:426-477", bins="i%H", node_size=[0, 10, n], trick=False,
                  parent_count=None, parent_sum=None, count=asym_c, sum=asym_s,
                  node_sum=None, total_sum=float(n * (n - 1) // 2)))
    h.append(dict(multi, name="MultiNodeHistSumDouble._2_NodesAsymmetricWithTrick",
                  cite="tests/cpp/test_hist_sum.cu:479-538", bins="i%H", node_size=[0, 10, n], trick=True,
                  parent_count=par_c, parent_sum=par_s, count=asym_c, sum=asym_s, node_sum=None))
    h.append(dict(multi, name="MultiNodeHistSumDouble._2_NodesAsymmetricWithTrick2",
                  cite="tests/cpp/test_hist_sum.cu:540-599", bins="i%H", node_size=[0, n - 10, n], trick=True,
                  parent_count=par_c, parent_sum=par_s,
                  count={str(i): v for i, v in enumerate([318, 318, 317, 317, 2, 2, 3, 3])},
                  sum={str(i): v for i, v in enumerate([201612.0, 201930.0, 200978.0, 201295.0, 2548.0, 2550.0,
                                                        3822.0, 3825.0])}, node_sum=None))
    h.append(dict(multi, name="MultiNodeHistSumDouble.SingleSegmentWithTrick",
                  cite="tests/cpp/test_hist_sum.cu:601-649", bins="0", node_size=[0, n // 2, n], trick=True,
                  parent_count=[n, 0, 0, 0], parent_sum=[float(n * (n - 1) // 2), 0.0, 0.0, 0.0],
                  count={"0": n // 2, "4": n // 2},
                  sum={"0": float((n // 2) * (n // 2 - 1) // 2), "4": float((n // 2) * (n // 2 + n - 1) // 2)},
                  node_sum=None))
    json.dump(h, open(os.path.join(HERE, "hist_sum.json"), "w"))
    print("fixtures written to", HERE)


if __name__ == "__main__":
    sys.exit(main())
