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
