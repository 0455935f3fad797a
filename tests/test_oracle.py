"""Pins the CPU oracle (oracle/nervanacpu.py) without running the reference.

Three kinds of checks: (1) the known answers and numpy restatements that the
reference's own tests hold, re-evaluated here through the oracle; (2)
brute-force scalar loops in pure Python/`math` on tiny inputs for every op,
broadcast class and reduction axis; (3) invariants that a dropped term, wrong
axis or transposed operand would break.
"""
import math

import numpy as np
import pytest

from neon_amd.backends.backend import Backend, OpTreeNode
from utils import assert_close, call_func, gen_inputs


# ---------------------------------------------------------------------------
# (1) golden vectors held by the reference's tests
# ---------------------------------------------------------------------------
def test_softmax_known_answer(cpu):
    """tests/test_activations.py:144-147: softmax of [0, 1, -2], tol 1e-7"""
    x = np.array([0, 1, -2], dtype=np.float32).reshape((3, 1))
    want = np.exp(x - 1) / np.sum(np.exp(x - 1))
    got = call_func(lambda be, t: be.fprop_softmax(t, 0), cpu, [x])
    assert np.allclose(got, want, atol=1e-7, rtol=0)
    # independent closed form
    e = [1.0, math.e, math.exp(-2)]
    assert np.allclose(got.ravel(), [v / sum(e) for v in e], atol=1e-7)


def test_softmax_big_inputs(cpu):
    """tests/test_activations.py:156-176: (1000, bsz=128) vs numpy, rtol 1e-5"""
    np.random.seed(1)
    x_ = np.random.random((1000, 128))
    x = cpu.iobuf(1000)
    x[:] = x_
    mx = np.max(x_, axis=0)
    ex = np.exp(x_ - mx)
    y_ = ex / np.sum(ex, axis=0)
    x[:] = cpu.fprop_softmax(x, 0)
    assert np.allclose(y_, x.get(), atol=0.0, rtol=1.0e-5)
    assert np.allclose(x.get().sum(axis=0), 1.0, atol=1e-5)


def _cross_entropy_multi(be, y, t):
    """CrossEntropyMulti.__call__ (neon/transforms/cost.py:159)"""
    return be.sum(-t * be.safelog(y), axis=0)


@pytest.mark.parametrize("outputs,targets,tol", [
    ([0.5, 0.9, 0.1, 0.0001], [0.5, 0.99, 0.01, 0.2], 1e-6),     # tests/test_costs.py:105-112
    ([0.5, 1.0, 0.0, 0.0001], [0.5, 0.0, 1.0, 0.2], 1e-5),       # tests/test_costs.py:115-122 (clamp)
])
def test_cross_entropy_multi_known_answers(cpu, outputs, targets, tol):
    y = np.array(outputs, dtype=np.float32).reshape((4, 1))
    t = np.array(targets, dtype=np.float32).reshape((4, 1))
    eps = np.exp(-50)
    want = np.sum(-np.array(targets) * np.log(np.maximum(np.array(outputs), eps)), keepdims=True).reshape(1, 1)
    got = call_func(_cross_entropy_multi, cpu, [y, t])
    assert np.allclose(got, want, atol=tol, rtol=0)
    if 0.0 in outputs:
        # log(0) clamped at exactly -50
        assert np.isclose(got[0, 0], 50.0 * 1.0 + (-0.5 * math.log(0.5)) - 0.2 * math.log(0.0001), atol=1e-4)


def test_misclassification_known_answer(cpu):
    """tests/test_costs.py:200-208: expected 1/3"""
    outputs = np.array([[0.25, 0.99, 0.33], [0.5, 0.005, 0.32], [0.25, 0.005, 0.34]], dtype=np.float32)
    targets = np.array([[0, 1, 0], [1, 0, 1], [0, 0, 0]], dtype=np.float32)
    be = cpu
    y, t = be.array(outputs), be.array(targets)
    preds, hyps, out = be.empty((1, 3)), be.empty((1, 3)), be.empty((1, 3))
    preds[:] = be.argmax(y, axis=0)                 # Misclassification.__call__, cost.py:421-425
    hyps[:] = be.argmax(t, axis=0)
    out[:] = be.not_equal(preds, hyps)
    assert np.isclose(out.get().mean(), 1.0 / 3.0, atol=1e-7)


def test_adam_step_matches_numpy_restatement(cpu):
    """tests/test_optimizer.py:280-299 with the reference's defaults, tol 1e-7"""
    from neon_amd import configs
    rs = np.random.RandomState(0)
    param = rs.rand(200, 128)
    grad = 0.01 * rs.rand(200, 128)
    states = [0.01 * rs.rand(200, 128), 0.01 * rs.rand(200, 128)]
    lr, b1, b2, eps = 0.001, 0.9, 0.999, 1e-8
    grad2 = grad / 128.
    m, v = states[0].copy(), states[1].copy()
    l = lr * np.sqrt(1. - b2 ** 1) / (1. - b1 ** 1)
    m[:] = m * b1 + (1. - b1) * grad2
    v[:] = v * b2 + (1. - b2) * grad2 * grad2
    want = param - l * m / (np.sqrt(v) + eps)

    be = cpu
    p = be.array(param.astype(np.float32))
    g = be.array(grad.astype(np.float32))
    tm, tv = be.array(states[0].astype(np.float32)), be.array(states[1].astype(np.float32))
    configs.c3_adam_step(be, p, g / 128., tm, tv, 1, lr, b1, b2, eps)
    assert p.dtype == np.float32 and p.get().dtype == np.float32
    assert np.allclose(p.get(), want, atol=1e-7, rtol=0)
    assert np.allclose(tm.get(), m, atol=1e-7) and np.allclose(tv.get(), v, atol=1e-9)


def test_scalar_subtrees_do_not_widen(cpu):
    """`lr * be.sqrt(1 - b2**t) / (1 - b1**t)` is a tree of numbers; its value
    must act like a Python float (numpy 1.13 value-based casting), i.e. an fp32
    tensor times it stays fp32 and equals the fp32 product."""
    be = cpu
    l = 1e-3 * be.sqrt(1 - 0.999 ** 3) / (1 - 0.9 ** 3)
    x = np.linspace(-1, 1, 12, dtype=np.float32).reshape(3, 4)
    t = be.array(x)
    out = be.empty((3, 4))
    out[:] = l * t
    lv = 1e-3 * math.sqrt(1 - 0.999 ** 3) / (1 - 0.9 ** 3)
    assert np.array_equal(out.get(), (x * np.float32(lv)).astype(np.float32))


def test_reduction_shapes(cpu):
    """tests/test_backend_autodiff_extra.py:250-261"""
    x0 = cpu.array(np.array([[1, 2], [4, 5]]), name="x0")
    assert cpu.sum(x0, axis=0).shape == (1, 2)
    assert cpu.sum(x0, axis=1).shape == (2, 1)
    assert cpu.sum(x0).shape == (1, 1)


def test_optree_printout(cpu):
    """doc/source/backends.rst:148-150"""
    x0 = cpu.array(np.ones((2, 2)), name="x0")
    x1 = cpu.array(np.ones((2, 2)), name="x1")
    f = x0 + x1
    assert isinstance(f, OpTreeNode)
    assert f[0] == {"shape": (2, 2), "op": "add"} and f[1] is x0 and f[2] is x1
    assert str(f) in ("({'shape': (2, 2), 'op': 'add'}, x0, x1)", "({'op': 'add', 'shape': (2, 2)}, x0, x1)")


# ---------------------------------------------------------------------------
# (2) brute force on tiny inputs
# ---------------------------------------------------------------------------
def _sig(x):
    return 1.0 / (1.0 + math.exp(-x))


UNARY_REF = {
    "negative": lambda x: -x, "absolute": abs,
    "sgn": lambda x: (x > 0) - (x < 0),
    "square": lambda x: x * x, "exp": math.exp, "exp2": lambda x: 2.0 ** x,
    "sig": _sig, "sig2": lambda x: 1.0 / (1.0 + 2.0 ** (-x)), "tanh": math.tanh,
    "tanh2": lambda x: (2.0 ** (2 * x) - 1) / (2.0 ** (2 * x) + 1),
    "rint": lambda x: float(round(x)),          # Python rounds half to even, like np.rint
}
UNARY_POS_REF = {"sqrt": math.sqrt, "log": math.log, "log2": math.log2,
                 "safelog": lambda x: math.log(max(x, math.exp(-50.0)))}


def test_unary_ops_bruteforce(cpu):
    vals = [-2.5, -1.0, -0.5, 0.0, 0.5, 1.5, 2.5, 3.25, -3.5, 0.125, 7.0, -0.0]
    x = np.array(vals, dtype=np.float32).reshape(4, 3)
    for name, f in UNARY_REF.items():
        got = call_func(lambda be, t, n=name: getattr(be, n)(t), cpu, [x])
        want = np.array([f(float(v)) for v in x.ravel()]).reshape(4, 3)
        assert np.allclose(got, want, rtol=2e-6, atol=1e-7), name
    xp = np.abs(x) + 0.01
    for name, f in UNARY_POS_REF.items():
        got = call_func(lambda be, t, n=name: getattr(be, n)(t), cpu, [xp])
        want = np.array([f(float(v)) for v in xp.ravel()]).reshape(4, 3)
        assert np.allclose(got, want, rtol=2e-6, atol=1e-7), name
    # safelog clamp: zero and a value below exp(-50) both give exactly -50
    tiny = np.array([[0.0, 1e-30, 1.0]], dtype=np.float32)
    got = call_func(lambda be, t: be.safelog(t), cpu, [tiny])
    assert np.allclose(got, [[-50.0, -50.0, 0.0]], atol=1e-5)
    assert call_func(lambda be, t: be.finite(t), cpu, [np.array([[1.0, np.inf, np.nan]], dtype=np.float32)]).tolist() \
        == [[1.0, 0.0, 0.0]]


BINARY_REF = {
    "add": lambda a, b: a + b, "subtract": lambda a, b: a - b, "multiply": lambda a, b: a * b,
    "divide": lambda a, b: a / b, "power": lambda a, b: abs(a) ** b,
    "maximum": max, "minimum": min,
    "equal": lambda a, b: float(a == b), "not_equal": lambda a, b: float(a != b),
    "less": lambda a, b: float(a < b), "less_equal": lambda a, b: float(a <= b),
    "greater": lambda a, b: float(a > b), "greater_equal": lambda a, b: float(a >= b),
}


@pytest.mark.parametrize("shapes", [((4, 3), (4, 3)), ((4, 3), (4, 1)), ((4, 3), (1, 3)),
                                    ((4, 1), (1, 3)), ((4, 3), (1, 1))])
def test_binary_ops_and_broadcast_bruteforce(cpu, shapes):
    rs = np.random.RandomState(3)
    a = np.round(rs.rand(*shapes[0]) * 4 - 2, 1).astype(np.float32)
    b = np.round(rs.rand(*shapes[1]) * 4 - 2, 1).astype(np.float32) + np.float32(2.5)
    R, C = max(shapes[0][0], shapes[1][0]), max(shapes[0][1], shapes[1][1])
    for name, f in BINARY_REF.items():
        if name == "power":
            got = call_func(lambda be, x, y: be.power(be.absolute(x), y), cpu, [a, b])
        else:
            got = call_func(lambda be, x, y, n=name: getattr(be, n)(x, y), cpu, [a, b])
        want = np.empty((R, C))
        for r in range(R):
            for c in range(C):
                av = float(a[r if shapes[0][0] > 1 else 0, c if shapes[0][1] > 1 else 0])
                bv = float(b[r if shapes[1][0] > 1 else 0, c if shapes[1][1] > 1 else 0])
                want[r, c] = f(av, bv)
        assert got.shape == (R, C), name
        assert np.allclose(got, want, rtol=2e-6, atol=1e-6), name


@pytest.mark.parametrize("axis", [0, 1])
def test_reductions_bruteforce(cpu, axis):
    x = np.array([[3, -1, 4, 1], [-5, 9, 2, 6], [5, 3, -5, 9]], dtype=np.float32)   # ties in max and min
    lines = [list(x[:, c]) for c in range(4)] if axis == 0 else [list(x[r, :]) for r in range(3)]
    shape = (1, 4) if axis == 0 else (3, 1)

    def ref(f):
        return np.array([f([float(v) for v in ln]) for ln in lines]).reshape(shape)
    n = len(lines[0])
    checks = {
        "sum": ref(sum), "max": ref(max), "min": ref(min),
        "mean": ref(lambda l: sum(l) / n),
        "var": ref(lambda l: sum((v - sum(l) / n) ** 2 for v in l) / n),
        "std": ref(lambda l: math.sqrt(sum((v - sum(l) / n) ** 2 for v in l) / n)),
        "argmax": ref(lambda l: l.index(max(l))), "argmin": ref(lambda l: l.index(min(l))),
    }
    for name, want in checks.items():
        got = call_func(lambda be, t, nm=name: getattr(be, nm)(t, axis=axis), cpu, [x])
        assert got.shape == shape
        assert np.allclose(got, want, rtol=1e-6, atol=1e-6), name


def test_argmax_first_occurrence(cpu):
    x = np.zeros((5, 6), dtype=np.float32)
    x[1, :] = 2
    x[3, :] = 2
    x[:, 4] = 2
    for axis, want in ((0, [1, 1, 1, 1, 0, 1]), (1, [4, 0, 4, 0, 4])):
        out = cpu.empty((1, 6) if axis == 0 else (5, 1), dtype=np.int32)
        out[:] = cpu.argmax(cpu.array(x), axis=axis)
        assert out.get().ravel().tolist() == want
        out[:] = cpu.argmin(cpu.array(-x), axis=axis)
        assert out.get().ravel().tolist() == want


def test_whole_tensor_reductions(cpu):
    x = gen_inputs(np.random.RandomState(5), (7, 9))
    assert np.isclose(call_func(lambda be, t: be.sum(t), cpu, [x])[0, 0], float(np.sum(x.astype(np.float64))), rtol=1e-5)
    assert call_func(lambda be, t: be.max(t), cpu, [x])[0, 0] == x.max()
    assert np.isclose(call_func(lambda be, t: be.mean(t), cpu, [x])[0, 0], x.mean(), rtol=1e-5, atol=1e-7)


def test_assign_casts(cpu):
    """numpy unsafe cast: float -> int truncates toward zero; fp32 -> fp16 rounds to nearest even"""
    x = np.array([[-1.7, -0.5, 0.5, 1.5, 2.5, 3.99]], dtype=np.float32)
    o = cpu.empty((1, 6), dtype=np.int32)
    o[:] = cpu.array(x) * 1.0
    assert o.get().tolist() == [[-1, 0, 0, 1, 2, 3]]
    h = cpu.empty((1, 2), dtype=np.float16)
    h[:] = cpu.array(np.array([[1.0 + 2 ** -11, 1.0 + 3 * 2 ** -11]], dtype=np.float32)) * 1.0
    assert h.get().tolist() == [[1.0, 1.0 + 2 ** -9]]      # ties to even


# ---------------------------------------------------------------------------
# one-hot: top-level form (reference) and the in-tree extension
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("axis", [0, 1])
def test_onehot_forms_agree(cpu, axis):
    rs = np.random.RandomState(9)
    n, k = 7, 5
    idx = rs.randint(0, k, (1, n)).astype(np.int32)
    shape = (k, n) if axis == 0 else (n, k)
    be = cpu
    ti = be.array(idx, dtype=np.int32)
    top = be.empty(shape)
    top[:] = be.onehot(ti, axis=axis)                       # reference form
    want = np.zeros(shape, dtype=np.float32)
    for j in range(n):
        if axis == 0:
            want[idx[0, j], j] = 1
        else:
            want[j, idx[0, j]] = 1
    assert np.array_equal(top.get(), want)
    y = be.array(rs.rand(*shape).astype(np.float32))
    a, b = be.empty(shape), be.empty(shape)
    a[:] = be.onehot(ti, axis=axis) * y + 1.0               # in-tree extension
    b[:] = top * y + 1.0
    assert np.array_equal(a.get(), b.get())


def test_hist_bruteforce(cpu):
    """Tensor.hist (tests/test_backend_hist.py:24-40): per-element binning done
    here with math.log2 and Python's round-half-even"""
    vals = [0.0, 1.0, 2.0, 3.0, -4.0, 1e-20, 1e30, 2.0 ** -48, 2.0 ** 16, 2.0 ** 15.4, -0.75, 6.0, 2.0 ** -47]
    a = np.array(vals, dtype=np.float32).reshape(1, -1)
    want = [0] * 64
    for v in a.ravel():
        v = abs(float(v))
        if v == 0.0:
            want[0] += 1
            continue
        b = round(math.log2(v)) + 48
        if b > 64:
            continue                    # beyond the last (closed) bin edge
        want[min(max(b, 0), 63)] += 1
    got = cpu.array(a).hist("t").get()
    assert got.shape == (1, 64) and got.ravel().tolist() == want


# ---------------------------------------------------------------------------
# views (tests/test_backend_tensor.py:252-315)
# ---------------------------------------------------------------------------
def test_views_alias_their_base(cpu):
    a = np.arange(24, dtype=np.float32).reshape(4, 6)
    t = cpu.array(a)
    for key in [0, -1, (0, slice(None)), slice(0, None), slice(None, -1), (slice(None), 0),
                (slice(None), slice(0, 1)), (-1, slice(0, None)), (slice(1, 3), slice(2, 5))]:
        v = t[key]
        want = a[key]
        want = want.reshape(v.shape)
        assert np.array_equal(v.get(), want), key
        assert len(v.shape) == 2
    t[1:3, 2:5] = 100.0
    a[1:3, 2:5] = 100.0
    t[:, 0] = t[:, 1] * 2.0
    a[:, 0] = a[:, 1] * 2.0
    assert np.array_equal(t.get(), a)
    assert np.array_equal(t.T.get(), a.T)
    assert np.array_equal(t.reshape((6, 4)).get(), a.reshape(6, 4))
    with pytest.raises(ValueError):
        t.reshape((5, 5))


# ---------------------------------------------------------------------------
# (3) invariants
# ---------------------------------------------------------------------------
def test_batchnorm_tree_invariants(cpu):
    from neon_amd import configs
    x, gamma, beta = configs.inputs_c4((6, 4096))
    be = cpu
    out = be.empty((6, 4096))
    configs.c4_rownorm(be, out, be.array(x.astype(np.float32)), be.array(gamma), be.array(beta))
    y = out.get().astype(np.float64)
    assert np.allclose(y.mean(axis=1), beta.ravel(), atol=1e-4)
    assert np.allclose(y.std(axis=1), gamma.ravel(), rtol=1e-4)
    v = call_func(lambda b, t: b.var(t, axis=1), cpu, [x.astype(np.float32)])
    assert (v >= 0).all()


def test_configs_against_float64_truth(cpu):
    """the oracle's own fp32 error on the benchmark trees (small instances)
    stays well inside the 1e-5 budget the device is held to"""
    from neon_amd import configs
    be = cpu
    (x2,) = configs.inputs_c2()
    o = be.empty(configs.C2_SHAPE)
    configs.c2_softmax(be, o, be.array(x2))
    x64 = x2.astype(np.float64)
    e = np.exp(x64 - x64.max(0))
    assert np.allclose(o.get(), e / e.sum(0), rtol=5e-6, atol=1e-30)
    x5, idx = configs.inputs_c5((2000, 64))
    t = be.empty((2000, 64))
    t[:] = be.onehot(be.array(idx, dtype=np.int32), axis=0)
    ce = be.empty((1, 64))
    configs.c5c_cross_entropy(be, ce, be.array(x5), t)
    x64 = x5.astype(np.float64)
    lse = np.log(np.exp(x64 - x64.max(0)).sum(0)) + x64.max(0)
    assert np.allclose(ce.get().ravel(), lse - x64[idx.ravel(), np.arange(64)], rtol=1e-5)
    am = be.empty((1, 64), dtype=np.int32)
    configs.c5a_argmax(be, am, be.array(x5))
    assert np.array_equal(am.get().ravel(), x5.argmax(axis=0))
    assert am.get().min() >= 0 and am.get().max() < 2000


def test_optree_node_utilities(cpu):
    """reflected power, !=, infix printing, list round trip, astensor /
    asnumpyarray, transpose of a node (reference backend.py:1893-2013)"""
    a = np.array([[1.0, 2.0], [3.0, 0.5]], dtype=np.float32)
    x = cpu.array(a, name="x")
    assert np.allclose((2.0 ** x).asnumpyarray(), 2.0 ** a)
    assert np.array_equal((x != 2.0).asnumpyarray(), (a != 2.0))
    tree = -(x * 2.0 + x ** 2.0)
    assert tree.pp() == "(neg ((x * (2.0)) + (x ** (2.0))))"
    assert str(x + 1.0) == "({'op': 'add', 'shape': (2, 2)}, x, 1.0)"
    lst = OpTreeNode.optree_to_list(tree)
    assert isinstance(lst, list) and lst[0]["op"] == "neg" and lst[2] is None and lst[1][1][1] is x
    back = OpTreeNode.list_to_optree(lst)
    assert isinstance(back, OpTreeNode) and np.array_equal(back.asnumpyarray(), tree.asnumpyarray())
    t = tree.astensor()
    assert t.shape == (2, 2) and np.allclose(t.get(), -(a * 2 + a ** 2))
    assert np.allclose((x * 2.0).transpose().asnumpyarray(), (a * 2).T)
    out = cpu.empty((2, 2))
    (x * 2.0).transpose(out=out)
    assert np.allclose(out.get(), (a * 2).T)
    with pytest.raises(ValueError):
        OpTreeNode.build("add", 1.0, 2.0).astensor()                # no tensor to take a backend from
    with pytest.raises(TypeError):
        x + "text"


def test_backend_base_helpers(cpu):
    """window arithmetic (reference backend.py:506-532 with the values its
    layers rely on), iobuf shapes, skip-node accumulation, compat mode"""
    from neon_amd.backends.backend import Backend
    assert cpu.output_dim(224, 7, 3, 2) == 112                      # (224 - 7 + 6) // 2 + 1
    assert cpu.output_dim(32, 3, 0, 1) == 30 and cpu.output_dim(32, 3, 1, 1) == 32
    assert cpu.output_dim(28, 3, 0, 1, dilation=2) == 24            # window widened to 5
    assert cpu.output_dim(13, 3, 0, 2, pooling=True) == 6
    with pytest.raises(ValueError):
        cpu.output_dim(13, 3, 3, 2, pooling=True)
    caffe = Backend.allocate_backend("cpu", rng_seed=0, compat_mode="caffe")
    assert caffe.check_caffe_compat() and not cpu.check_caffe_compat()
    assert caffe.output_dim(14, 3, 0, 2, pooling=True) == 7         # ceil((14 - 3) / 2) + 1; plain floor gives 6
    assert caffe.output_dim(14, 3, 0, 2) == 6                       # convolutions keep the floor
    assert caffe.output_dim(8, 3, 1, 2, pooling=True) == 5 and caffe.output_dim(7, 2, 1, 2, pooling=True) == 4
    with pytest.raises(ValueError):
        Backend.allocate_backend("cpu", rng_seed=0, compat_mode="other")
    bsz = cpu.bsz
    assert cpu.iobuf(10).shape == (10, bsz) and cpu.iobuf((10, 4)).shape == (10, 4 * bsz)
    assert cpu.iobuf((3, 4, 5)).shape == (60, bsz)
    given = cpu.empty((2, 2))
    assert cpu.iobuf(10, x=given) is given
    pool = cpu.zeros((20, bsz))
    shared = cpu.iobuf(10, shared=pool)
    assert shared.shape == (10, bsz) and not shared.get().any()
    x, y = cpu.array(np.full((3, 2), 2.0, np.float32)), cpu.array(np.full((3, 2), 5.0, np.float32))
    cpu.fprop_skipnode(x, y, beta=0.5)
    assert np.array_equal(y.get(), np.full((3, 2), 4.5))
    d = cpu.array(np.full((3, 2), 1.0, np.float32))
    cpu.bprop_skipnode(x, d, alpha=3.0, beta=2.0)
    assert np.array_equal(d.get(), np.full((3, 2), 8.0))
    state = cpu.rng_get_state()
    first = cpu.rng.uniform(size=3)
    cpu.rng_set_state(state)
    assert np.array_equal(cpu.rng.uniform(size=3), first)
    cpu.rng_reset()


# ---- bfloat16 rounding (oracle/bf16.py) -------------------------------------------------------
def test_bf16_rounding_is_pinned_bit_for_bit():
    """exhaustive over the bf16 values and their neighbourhoods, exact rational
    arithmetic on a sample, and agreement with the product's bit trick"""
    from fractions import Fraction
    from oracle.bf16 import round_to_bf16
    from neon_amd.backends.hip import bf16 as product
    # every bf16 value is a fixed point; so is its float32 image
    all_bf16 = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    finite = np.isfinite(all_bf16)
    assert np.array_equal(round_to_bf16(all_bf16[finite]).view(np.uint32), all_bf16[finite].view(np.uint32))
    # halfway points: ties go to the even neighbour; one float32 step either side goes to the nearer one
    base = (np.arange(0x0080, 0x7F7F, dtype=np.uint32) << 16)                  # positive normal bf16 values
    for sign in (0, 0x80000000):
        b = base | np.uint32(sign)
        tie = (b | np.uint32(0x8000)).view(np.float32)
        lower_even = ((b >> 16) & 1) == 0
        want = np.where(lower_even, b, b + np.uint32(0x10000))
        assert np.array_equal(round_to_bf16(tie).view(np.uint32), want)
        assert np.array_equal(round_to_bf16((b | np.uint32(0x7FFF)).view(np.float32)).view(np.uint32), b)
        assert np.array_equal(round_to_bf16((b | np.uint32(0x8001)).view(np.float32)).view(np.uint32),
                              b + np.uint32(0x10000))
    # overflow, infinities, NaN, zeros, denormals
    top = np.array([0x7F7F8000, 0x7F7F7FFF, 0x7F7FFFFF], dtype=np.uint32).view(np.float32)
    assert np.array_equal(round_to_bf16(top).view(np.uint32), np.array([0x7F800000, 0x7F7F0000, 0x7F800000], np.uint32))
    special = np.array([np.inf, -np.inf, 0.0, -0.0, 1e-40, -3e-41], dtype=np.float32)
    got = round_to_bf16(special)
    assert np.array_equal(got[:4].view(np.uint32), special[:4].view(np.uint32))
    assert np.isnan(round_to_bf16(np.array([np.nan], np.float32)))[0]
    # exact rational check of "nearest, ties to even" on random float32 values
    rs = np.random.RandomState(5)
    sample = (rs.standard_normal(400) * np.exp(rs.uniform(-60, 60, 400))).astype(np.float32)
    sample = np.concatenate([sample, special[4:]])
    for x, r in zip(sample, round_to_bf16(sample)):
        fx, fr = Fraction(float(x)), Fraction(float(r))
        b = int(np.array([r], np.float32).view(np.uint32)[0])
        assert b & 0xFFFF == 0                                              # a bf16 value
        for nb in (b - 0x10000, b + 0x10000):                               # no neighbour is nearer
            if 0 <= (nb & 0x7FFFFFFF) < 0x7F800000 and (nb ^ b) >> 31 == 0:
                other = Fraction(float(np.array([nb], np.uint32).view(np.float32)[0]))
                assert abs(fx - fr) <= abs(fx - other)
                if abs(fx - fr) == abs(fx - other):
                    assert (b >> 16) & 1 == 0
    # the product's host conversion (add-and-shift) agrees bit for bit, and so do the widening helpers
    big = (rs.standard_normal(200000) * np.exp(rs.uniform(-80, 80, 200000))).astype(np.float32)
    big = np.concatenate([big, all_bf16[finite], top, special])
    assert np.array_equal(product.quantise(big).view(np.uint32), round_to_bf16(big).view(np.uint32))
    assert np.array_equal(product.from_bits(product.to_bits(big)), product.quantise(big))
