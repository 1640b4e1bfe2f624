"""The scikit-learn style estimators (python-package/arboretum/core.py:342-732 of the reference):
the reference's classifier golden (tests/py/test_sklearn_classification.py:9-61) and the
early-stopping loop of fit() (core.py:435-507)."""
import numpy as np
import pytest

from conftest import load_golden

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def arb():
    import arboretum_amd
    if arboretum_amd.device_count() < 1:
        pytest.fail("no HIP device: the GPU tests must run on the GPU box")
    return arboretum_amd


FX = load_golden("sklearn_classification_iris.json")


@pytest.mark.parametrize("double_precision", FX["sweep"]["double_precision"])
@pytest.mark.parametrize("hist_size", FX["sweep"]["hist_size"])
def test_classifier_golden(arb, double_precision, hist_size):
    X = np.array(FX["X"], np.float32)
    y = np.array(FX["target"]) != 2                     # the test's label rule, a bool array as there
    params = {k: v for k, v in FX["params"].items() if not (isinstance(v, str) and v.startswith("$"))}
    model = arb.ArboretumClassifier(double_precision=double_precision, method="hist", hist_size=hist_size, **params)
    data = arb.DMatrix(X, y=y)
    model.fit(data, y)
    assert np.allclose(model.predict(data), FX["y_pred"])


def _problem(n, seed):
    rng = np.random.default_rng(seed)
    X = rng.normal(size=(n, 6)).astype(np.float32)
    signal = X[:, 0] * X[:, 1] + np.sin(2 * X[:, 2])
    return X, signal, rng


def test_early_stopping_follows_the_reference_loop(arb):
    # regression on a small noisy training set: the evaluation error goes through a minimum; fit()
    # must stop early_stopping_rounds rounds after the best round, keep best_round / best_score, and
    # the evaluation predictions it tracked with append_last_tree must equal a fresh predict()
    X, signal, rng = _problem(400, 3)
    y = (signal + 1.5 * rng.normal(size=400)).astype(np.float32)
    Xe, se, _ = _problem(3000, 4)
    ye = se.astype(np.float32)
    scores = []

    def mse(labels, pred):
        scores.append(float(np.mean((labels - pred) ** 2)))
        return scores[-1]
    model = arb.ArboretumRegression(max_depth=5, learning_rate=0.5, n_estimators=200, verbosity=0, l1=0, l2=0.1,
                                    colsample_bytree=1.0, min_child_weight=1.0, hist_size=63, double_precision=True)
    eval_data = arb.DMatrix(Xe)
    model.fit(X, y, eval_set=eval_data, eval_labels=ye, early_stopping_rounds=4, eval_metric=mse)
    rounds = len(scores)
    assert rounds < 200, "the evaluation error never stopped improving"
    best = int(np.argmin(scores))
    # the loop's rule: stop at the first i with early_stopping_rounds + best_round < i
    assert model.best_round == best and model.best_score == scores[best]
    assert rounds - 1 == best + 4 + 1
    assert all(s >= scores[best] for s in scores[best:])
    # every round's score is the metric of the predictions after exactly that many trees
    g = model._garden
    assert g.num_trees() == rounds
    for r in (1, best + 1, rounds):
        assert np.isclose(np.mean((ye - g.predict(eval_data, n_rounds=r)) ** 2), scores[r - 1], rtol=1e-5)
    # best_round selects the model to predict with
    assert np.array_equal(model.predict(eval_data, n_rounds=model.best_round + 1), g.predict(eval_data, n_rounds=best + 1))


def test_without_an_evaluation_set_every_round_is_grown(arb):
    X, signal, rng = _problem(300, 5)
    y = (signal > 0)
    model = arb.ArboretumClassifier(max_depth=3, learning_rate=0.3, n_estimators=7, verbosity=0, colsample_bytree=1.0)
    model.fit(X, y.astype(np.float32))
    assert model._garden.num_trees() == 7 and model.best_round == -1
    p = model.predict(X)
    assert p.shape == (300,) and ((p > 0.5) == y).mean() > 0.8


def test_classifier_early_stopping_with_the_default_metric(arb):
    X, signal, rng = _problem(500, 7)
    y = (signal + 1.0 * rng.normal(size=500) > 0).astype(np.float32)
    Xe, se, _ = _problem(2000, 8)
    ye = (se > 0).astype(np.float32)
    model = arb.ArboretumClassifier(max_depth=4, learning_rate=0.5, n_estimators=150, verbosity=0, l2=0.1,
                                    colsample_bytree=1.0)
    model.fit(X, y, eval_set=Xe, eval_labels=ye, early_stopping_rounds=3)
    n = model._garden.num_trees()
    assert n < 150 and n - 1 == model.best_round + 3 + 1
    assert np.isfinite(model.best_score)
