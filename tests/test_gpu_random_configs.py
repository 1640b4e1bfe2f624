"""Seeded random configurations of the HIP path against the oracle: shapes,
objectives and parameters drawn at random, every intermediate compared bit for
bit (the comparison itself lives in test_gpu_parity.assert_same_training)."""
import os

import numpy as np
import pytest

from test_gpu_parity import assert_same_training, make_data

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


def _draw(seed):
    rng = np.random.default_rng(1000 + seed)
    objective = int(rng.integers(0, 2))
    n = int(rng.choice([37, 300, 2049, 9000, 33000, 70000]))
    F = int(rng.choice([1, 2, 3, 5, 8, 13, 28, 31, 33, 40]))
    depth = int(rng.integers(1, 8))
    hist_size = int(rng.choice([2, 7, 16, 63, 64, 100, 255, 256, 300, 1000]))
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": hist_size, "double_precision": bool(rng.integers(0, 2)),
                         "use_hist_subtraction_trick": bool(rng.integers(0, 2)),
                         # 16-bit bins (more than 257 ids per feature) are resident only; 256 thresholds
                         # and a bin for missing values stay on the 8-bit kernels, streamed too
                         "upload_features": bool(rng.random() < 0.75) or hist_size > 256,
                         "stream_block_rows": int(rng.choice([64, 1000, 5000, 1 << 20])),
                         "seed": int(rng.integers(0, 100))},
           "tree": {"max_depth": depth, "eta": float(rng.choice([0.1, 0.3, 1.0])),
                    "lambda": float(rng.choice([0.0, 0.5, 1.0, 3.0])),
                    "alpha": float(rng.choice([0.0, 0.0, 0.2])),
                    "min_child_weight": float(rng.choice([0.0, 1.0, 5.0])),
                    "min_leaf_size": int(rng.choice([0, 1, 10])),
                    "gamma_absolute": float(rng.choice([0.0, 0.0, 0.1])),
                    "colsample_bytree": float(rng.choice([1.0, 1.0, 0.8])),
                    "colsample_bylevel": float(rng.choice([1.0, 1.0, 0.7]))}}
    nan_frac = float(rng.choice([0.0, 0.0, 0.02, 0.3]))
    inspect = bool(rng.random() < 0.6)
    return n, F, objective, cfg, nan_frac, inspect


@pytest.mark.parametrize("seed", range(int(os.environ.get("ARB_SEEDS", "64"))))
def test_random_configuration(arb, oracle, seed):
    n, F, objective, cfg, nan_frac, inspect = _draw(seed)
    columns = F
    if int(cfg["tree"]["colsample_bytree"] * columns) == 0 or \
            int(cfg["tree"]["colsample_bytree"] * cfg["tree"]["colsample_bylevel"] * columns) == 0:
        cfg["tree"]["colsample_bytree"] = cfg["tree"]["colsample_bylevel"] = 1.0
    X, y = make_data(n, F, objective, seed=seed, nan_frac=nan_frac)
    assert_same_training(arb, oracle, X, y, cfg, rounds=3, check_hist=inspect)


def _draw_wide(seed):
    """Matrices wider than one LDS histogram: rows in place as records (one launch when the bins in
    use fit one histogram, groups of 32 features otherwise), or the row-moving group passes."""
    rng = np.random.default_rng(5000 + seed)
    objective = int(rng.integers(0, 2))
    n = int(rng.choice([63, 1000, 4097, 30000]))
    F = int(rng.choice([33, 36, 64, 70, 100, 130, 200, 260]))
    depth = int(rng.integers(2, 8))
    hist_size = int(rng.choice([7, 31, 63, 100, 255, 256]))
    cfg = {"objective": objective, "method": 1,
           "internals": {"hist_size": hist_size, "double_precision": bool(rng.integers(0, 2)),
                         "use_hist_subtraction_trick": bool(rng.integers(0, 2)),
                         "wide_rows_in_place": bool(rng.random() < 0.8),
                         "seed": int(rng.integers(0, 100))},
           "tree": {"max_depth": depth, "eta": float(rng.choice([0.1, 0.3, 1.0])),
                    "lambda": float(rng.choice([0.0, 0.5, 1.0, 3.0])),
                    "min_child_weight": float(rng.choice([0.0, 1.0, 5.0])),
                    "min_leaf_size": int(rng.choice([0, 1, 10])),
                    "colsample_bytree": float(rng.choice([1.0, 1.0, 0.8])),
                    "colsample_bylevel": float(rng.choice([1.0, 1.0, 0.7]))}}
    nan_frac = float(rng.choice([0.0, 0.02, 0.3]))
    inspect = bool(rng.random() < 0.5) and n * F < 2_000_000
    return n, F, objective, cfg, nan_frac, inspect


@pytest.mark.parametrize("seed", range(int(os.environ.get("ARB_WIDE_SEEDS", "32"))))
def test_random_wide_configuration(arb, oracle, seed):
    n, F, objective, cfg, nan_frac, inspect = _draw_wide(seed)
    X, y = make_data(n, F, objective, seed=seed, nan_frac=nan_frac)
    assert_same_training(arb, oracle, X, y, cfg, rounds=2, check_hist=inspect)
