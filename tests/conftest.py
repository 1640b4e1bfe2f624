import json
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def load_golden(name):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)


def concrete_config(template, **subst):
    """Replaces the "$name" placeholders of a fixture's config template."""
    def ev(v):
        if isinstance(v, dict):
            return {k: ev(x) for k, x in v.items()}
        if isinstance(v, str) and v.startswith("$"):
            return subst[v[1:]]
        return v
    return ev(template)


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as orc
    orc.lib()
    return orc


def hist_sum_inputs(case):
    """Inputs of one tests/cpp/test_hist_sum.cu case: one feature column of bin ids, grad[i] = i,
    node offsets."""
    import numpy as np
    n, H = case["rows"], case["hist_size"]
    i = np.arange(n)
    bins = {"i": i, "0": np.zeros(n, np.int64), "i%H": i % H}[case["bins"]].astype(np.uint8)
    return bins.reshape(n, 1), i.astype(np.float32), np.array(case["node_size"], np.uint32)


def check_hist_sum(case, count, total):
    """count, total: [nodes][>= hist_size] arrays of row counts and gradient sums."""
    import numpy as np
    H = case["hist_size"]
    for k, v in case["count"].items():
        assert count[int(k) // H][int(k) % H] == v, (case["name"], "count", k)
    for k, v in case["sum"].items():
        assert total[int(k) // H][int(k) % H] == v, (case["name"], "sum", k)
    if case.get("node_sum"):
        for nd, v in enumerate(case["node_sum"]):
            assert float(np.sum(total[nd][:H])) == v, (case["name"], "node_sum", nd)
    if case.get("total_sum") is not None:
        assert float(np.sum(np.asarray(total)[:, :H])) == case["total_sum"]
