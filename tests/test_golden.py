"""The committed known-answer fixture (tests/golden/known_answers.json: cases
the reference's own tests hold, written by tests/golden/make_known_answers.py)
against the oracle on the CPU and against the hip backend on the GPU."""
import contextlib
import json
import os

import numpy as np
import pytest

from neon_amd import NervanaObject
from neon_amd.backends.autodiff import Autodiff
from neon_amd.optimizers import Adam
from neon_amd.transforms import (CrossEntropyBinary, CrossEntropyMulti, Logistic, MeanSquared,
                                 Misclassification, PrecisionRecall, Rectlin, Softmax, SumSquared, Tanh)

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "known_answers.json")) as _f:
    CASES = json.load(_f)["cases"]


@contextlib.contextmanager
def _using(be, bsz):
    old, old_bsz = NervanaObject.be, be.bsz
    NervanaObject.be, be.bsz = be, bsz
    try:
        yield
    finally:
        NervanaObject.be, be.bsz = old, old_bsz


class _Layer(object):
    def __init__(self, plist):
        self.plist = plist

    def get_params(self):
        return self.plist


def _evaluate(be, case):
    kind = case["kind"]
    arrays = [np.asarray(a, dtype=np.float32) for a in case["inputs"]]
    tensors = [be.array(a) for a in arrays]
    batch = arrays[0].shape[1]
    with _using(be, batch):
        act = {"softmax_axis0": lambda: Softmax(), "tanh": lambda: Tanh(), "sig": lambda: Logistic(),
               "relu": lambda: Rectlin(slope=case.get("slope", 0))}
        cost = {"ce_binary": CrossEntropyBinary, "ce_multi": CrossEntropyMulti, "sum_squared": SumSquared,
                "mean_squared": MeanSquared}
        if kind in act:
            tree = act[kind]()(tensors[0])
            out = be.empty(tree.shape)
            out[:] = tree
            return out.get()
        if kind in cost:
            tree = cost[kind]()(*tensors)
            out = be.empty(tree.shape)
            out[:] = tree
            return out.get()
        if kind == "misclassification":
            return np.array([[Misclassification()(*tensors)]])
        if kind == "precision_recall":
            return PrecisionRecall(arrays[0].shape[0])(*tensors)
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
            opt = Adam(learning_rate=prm["lr"], beta_1=prm["beta_1"], beta_2=prm["beta_2"], epsilon=prm["epsilon"])
            opt.be = be
            opt.optimize([_Layer([((p, g), [m, v])])], epoch=0)
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
