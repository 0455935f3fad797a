"""The committed known-answer fixture (tests/golden/known_answers.json: cases
the reference's own tests hold, written by tests/golden/make_known_answers.py)
against the oracle on the CPU and against the hip backend on the GPU."""
import contextlib
import json
import os

import numpy as np
import pytest

from neon_amd.backends.autodiff import Autodiff
import clients

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")) as _f:
    CASES = json.load(_f)["cases"]


@contextlib.contextmanager
def _batch(be, bsz):
    old = be.bsz
    be.bsz = bsz
    try:
        yield
    finally:
        be.bsz = old


def _evaluate(be, case):
    kind = case["kind"]
    arrays = [np.asarray(a, dtype=np.float32) for a in case["inputs"]]
    tensors = [be.array(a) for a in arrays]
    trees = {"softmax_axis0": clients.softmax, "tanh": clients.tanh, "sig": clients.logistic,
             "relu": lambda be_, x: clients.rectlin(be_, x, case.get("slope", 0)),
             "ce_binary": clients.cross_entropy_binary, "ce_multi": clients.cross_entropy_multi,
             "sum_squared": clients.sum_squared, "mean_squared": clients.mean_squared}
    with _batch(be, arrays[0].shape[1]):
        if kind in trees:
            tree = trees[kind](be, *tensors)
            out = be.empty(tree.shape)
            out[:] = tree
            return out.get()
        if kind == "misclassification":
            return np.array([[clients.misclassification(be, *tensors)]])
        if kind == "precision_recall":
            return clients.precision_recall(be, *tensors)
        if kind == "autodiff_poly":
            x0, x1, x2, x3 = tensors
            f = x0 * x0 - x1 * x0 + x0 * x2 - x2 * x1 * x0 + x3 * x3 * x3
            grads = Autodiff(f, be).get_grad_asnumpyarray(tensors)
            for g in grads:
                assert np.all(g == g[0, 0])
            return np.array([g[0, 0] for g in grads])
        if kind == "adam":
            prm = case["params"]
            be.bsz = prm["bsz"]
            p, g, m, v = tensors
            clients.adam_update(be, p, g, m, v, 1, lr=prm["lr"], b1=prm["beta_1"], b2=prm["beta_2"],
                                eps=prm["epsilon"])
            return p.get()
    raise AssertionError("unknown case kind %s" % kind)


def _check(be, case):
    got = np.asarray(_evaluate(be, case), dtype=np.float64)
    want = np.asarray(case["expected"], dtype=np.float64)
    assert got.shape == want.shape, (case["name"], got.shape, want.shape)
    assert np.all(np.abs(got - want) <= case["tol"] + 1e-12), (case["name"], got, want)


@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_known_answers_oracle(cpu, case):
    _check(cpu, case)


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES, ids=[c["name"] for c in CASES])
def test_known_answers_hip(hip, case):
    _check(hip, case)
