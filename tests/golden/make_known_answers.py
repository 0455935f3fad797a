"""Writes tests/golden/known_answers.json: the known-answer cases that the
reference's own test files hold for the op-tree path, as plain data (inputs
and expected outputs).  Nothing of the reference is imported or run: every
expected value is either a literal of the cited test or the float64 numpy
evaluation of the closed form that test states.

    python tests/golden/make_known_answers.py
"""
import json
import os

import numpy as np

EPS = np.exp(-50)
cases = []


def add(name, source, kind, inputs, expected, tol, **extra):
    entry = {"name": name, "source": source, "kind": kind,
             "inputs": [np.asarray(a, dtype=np.float64).tolist() for a in inputs],
             "expected": np.asarray(expected, dtype=np.float64).tolist(), "tol": tol}
    entry.update(extra)
    cases.append(entry)


col = lambda *v: np.array(v, dtype=np.float64).reshape((-1, 1))
x = col(0, 1, -2)

# activations: tests/test_activations.py
add("softmax", "tests/test_activations.py:144-147", "softmax_axis0", [x], np.exp(x - 1) / np.sum(np.exp(x - 1)), 1e-7)
add("tanh", "tests/test_activations.py:208-212", "tanh", [x], np.tanh(x), 1e-7)
add("logistic", "tests/test_activations.py:229-232", "sig", [x], 1.0 / (1.0 + np.exp(-x)), 1e-7)
add("rectlin_mixed", "tests/test_activations.py:73-76", "relu", [[[4, 0], [-2, 9]]], [[4, 0], [0, 9]], 0.0, slope=0.0)
add("leaky_rectlin_mixed", "tests/test_activations.py:112-116", "relu", [[[4, 0], [-2, 9]]], [[4, 0], [-0.4, 9]], 1e-7,
    slope=0.2)

# costs: tests/test_costs.py
y1, t1 = col(0.5, 0.9, 0.1, 0.0001), col(0.5, 0.99, 0.01, 0.2)
y2, t2 = col(0.5, 1.0, 0.0, 0.0001), col(0.5, 0.0, 1.0, 0.2)
for tag, y, t, tol, src in (("", y1, t1, 1e-6, "66-75"), ("_limits", y2, t2, 1e-5, "78-87")):
    add("cross_entropy_binary" + tag, "tests/test_costs.py:" + src, "ce_binary", [y, t],
        np.sum(-t * np.log(np.maximum(y, EPS)) - (1 - t) * np.log(np.maximum(1 - y, EPS)), keepdims=True), tol)
for tag, y, t, tol, src in (("", y1, t1, 1e-6, "105-112"), ("_limits", y2, t2, 1e-5, "115-122")):
    add("cross_entropy_multi" + tag, "tests/test_costs.py:" + src, "ce_multi", [y, t],
        np.sum(-t * np.log(np.maximum(y, EPS)), axis=0, keepdims=True), tol)
add("sum_squared", "tests/test_costs.py:138-142", "sum_squared", [y1, t1],
    np.sum((y1 - t1) ** 2, axis=0, keepdims=True) / 2.0, 1e-7)
add("mean_squared", "tests/test_costs.py:165-169", "mean_squared", [y1, t1],
    np.mean((y1 - t1) ** 2, axis=0, keepdims=True) / 2.0, 1e-7)
add("misclassification", "tests/test_costs.py:200-207", "misclassification",
    [[[0.25, 0.99, 0.33], [0.5, 0.005, 0.32], [0.25, 0.005, 0.34]], [[0, 1, 0], [1, 0, 1], [0, 0, 0]]], [[1.0 / 3]], 1e-7)
add("precision_recall", "tests/test_costs.py:215-221", "precision_recall",
    [[[0, 1, 0, 1], [1, 0, 0, 0], [0, 0, 1, 0]], [[0, 1, 0, 1], [1, 0, 1, 0], [0, 0, 0, 0]]],
    np.array([1 + 1 + 0, 1 + 0.5 + 0]) / 3.0, 1e-6)

# autodiff: tests/test_backend_autodiff_extra.py:358-379 (x0..x3 = 1, 2, 3, 5 on 3x3;
# f = x0*x0 - x1*x0 + x0*x2 - x2*x1*x0 + x3*x3*x3)
add("autodiff_hard_coded", "tests/test_backend_autodiff_extra.py:358-379", "autodiff_poly",
    [np.full((3, 3), v) for v in (1, 2, 3, 5)], [-3.0, -4.0, -1.0, 75.0], 1e-5)

# one Adam step, tests/test_optimizer.py:280-299 (closed form; batch size 128)
rs = np.random.RandomState(0)
p, g = rs.rand(6, 4), 0.01 * rs.rand(6, 4)
m0, v0 = 0.01 * rs.rand(6, 4), 0.01 * rs.rand(6, 4)
lr, b1, b2, eps, t = 0.001, 0.9, 0.999, 1e-8, 1
gg = g / 128.0
m = m0 * b1 + (1 - b1) * gg
v = v0 * b2 + (1 - b2) * gg * gg
add("adam_step", "tests/test_optimizer.py:280-299", "adam", [p, g, m0, v0],
    p - (lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t)) * m / (np.sqrt(v) + eps), 1e-6,
    params={"lr": lr, "beta_1": b1, "beta_2": b2, "epsilon": eps, "bsz": 128})

here = os.path.dirname(os.path.abspath(__file__))
with open(os.path.join(here, "known_answers.json"), "w") as f:
    f.write('{"cases": [\n' + ",\n".join(json.dumps(c) for c in cases) + "\n]}\n")
print("wrote %d cases" % len(cases))
