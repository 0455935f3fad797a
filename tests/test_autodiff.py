"""Gradients of op-trees (neon_amd/backends/autodiff.py).

Pins, in order: the reference's own known-answer test (tests/test_autodiff.py
``test_hard_coded``: closed-form gradients of a polynomial), central finite
differences of an independent float64 numpy evaluation of each function, and --
on the GPU -- the hip backend's gradients against the oracle backend's for the
same trees, including the reference's batch-norm tree with an incoming error.
"""
import numpy as np
import pytest

from neon_amd.backends.autodiff import Autodiff
from utils import assert_close


class _NP(object):
    """float64 numpy stand-in for the handful of backend builders the test
    functions use, so finite differences do not go through the code under test"""
    @staticmethod
    def sum(a, axis=None):
        return np.sum(a, axis=axis, keepdims=True)

    @staticmethod
    def max(a, axis=None):
        return np.max(a, axis=axis, keepdims=True)

    @staticmethod
    def min(a, axis=None):
        return np.min(a, axis=axis, keepdims=True)

    @staticmethod
    def mean(a, axis=None):
        return np.mean(a, axis=axis, keepdims=True)

    @staticmethod
    def var(a, axis=None):
        return np.var(a, axis=axis, keepdims=True)

    @staticmethod
    def std(a, axis=None):
        return np.std(a, axis=axis, keepdims=True)

    @staticmethod
    def argmax(a, axis=1):
        return np.argmax(a, axis=axis).reshape((-1, 1) if axis == 1 else (1, -1))

    @staticmethod
    def argmin(a, axis=1):
        return np.argmin(a, axis=axis).reshape((-1, 1) if axis == 1 else (1, -1))

    exp = staticmethod(np.exp)
    log = staticmethod(np.log)
    tanh = staticmethod(np.tanh)
    sqrt = staticmethod(np.sqrt)
    square = staticmethod(np.square)
    absolute = staticmethod(np.abs)
    maximum = staticmethod(np.maximum)
    minimum = staticmethod(np.minimum)
    exp2 = staticmethod(np.exp2)
    log2 = staticmethod(np.log2)

    @staticmethod
    def sig(a):
        return 1.0 / (1.0 + np.exp(-a))

    @staticmethod
    def transpose(a):
        return a.T


def _T(ns, a):
    return ns.transpose(a) if isinstance(ns, _NP) else a.T


# (name, f(ns, *xs), operand shapes, kind of inputs)
FUNCS = [
    ("poly", lambda ns, a, b, c: a * a - b * a + a * c - c * b * a + b * b * b, [(6, 9)] * 3, "rand"),
    ("divide", lambda ns, a, b: a / (b + 2.0) - 3.0 / (a + 2.0), [(5, 7)] * 2, "pos"),
    ("unary", lambda ns, a, b: ns.exp(a) * ns.tanh(b) + ns.sig(a * b) - ns.log(b + 2.0) + ns.sqrt(a + 3.0),
     [(6, 5)] * 2, "rand"),
    ("base2", lambda ns, a, b: ns.exp2(a) + ns.log2(b + 2.0) * a, [(4, 6)] * 2, "rand"),
    ("sqr_abs_neg", lambda ns, a, b: ns.square(a) * ns.absolute(b) + (-a) * b, [(4, 8)] * 2, "rand"),
    ("power", lambda ns, a, b: (a + 2.0) ** (b + 1.5), [(5, 5)] * 2, "pos"),
    ("maxmin", lambda ns, a, b: ns.maximum(a, b) * 2.0 + ns.minimum(a, b * b), [(7, 6)] * 2, "rand"),
    ("bcast_col", lambda ns, a, b: a * b + b, [(6, 9), (6, 1)], "rand"),
    ("bcast_row", lambda ns, a, b: a / (b + 2.0) + a * b, [(6, 9), (1, 9)], "rand"),
    ("bcast_scalar", lambda ns, a, b: ns.tanh(a * b) + b, [(5, 4), (1, 1)], "rand"),
    ("sum_axis1", lambda ns, a, b: ns.sum(a * b, axis=1) * ns.sum(a, axis=1), [(6, 9)] * 2, "rand"),
    ("sum_axis0", lambda ns, a, b: a * ns.sum(ns.exp(a) * b, axis=0), [(6, 9)] * 2, "rand"),
    ("sum_all", lambda ns, a, b: ns.sum(a * b) * a, [(5, 6)] * 2, "rand"),
    ("max_axis", lambda ns, a, b: ns.max(a, axis=1) * b + ns.min(b, axis=0) * a, [(6, 9)] * 2, "rand"),
    ("mean_var", lambda ns, a, b: (a - ns.mean(a, axis=1)) / ns.sqrt(ns.var(a, axis=1) + 1e-3) * b,
     [(8, 12)] * 2, "rand"),
    ("softmax", lambda ns, a: ns.exp(a - ns.max(a, axis=0)) / ns.sum(ns.exp(a - ns.max(a, axis=0)), axis=0)
     * ns.exp(a), [(10, 6)], "rand"),
    # reference tests/test_backend_autodiff_extra.py test_reduction: every reduction, with and without an axis
    ("reduction_mix", lambda ns, a, b, c, d: (a + c) + ns.sum(a, axis=0) - (a - b) - ns.mean(d, axis=1)
     + (c + d) + ns.var(a, axis=0) + (c + d) + ns.std(a) - (c - d) - ns.max(d, axis=1)
     - (c - d) - ns.min(d, axis=0) - (c - d) - ns.argmax(d, axis=1) - (c - d) - ns.argmin(d, axis=0),
     [(5, 7)] * 4, "rand"),
    # transposes of op-trees (a transposed *tensor* is a view and is keyed by its base)
    ("transpose", lambda ns, a, b: _T(ns, a * 2.0) * b + _T(ns, _T(ns, b * b) * a), [(5, 8), (8, 5)], "rand"),
]
IDS = [f[0] for f in FUNCS]


def _inputs(shapes, kind, seed):
    rs = np.random.RandomState(seed)
    if kind == "pos":
        return [(0.5 + rs.rand(*s)).astype(np.float32) for s in shapes]
    return [(-1 + 2 * rs.rand(*s)).astype(np.float32) for s in shapes]


def _numerical(f, arrays, err, h=1e-6):
    """d sum(f*err) / d arrays[i] by central differences in float64"""
    xs = [a.astype(np.float64) for a in arrays]
    grads = []
    for x in xs:
        g = np.zeros_like(x)
        it = np.nditer(x, flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            keep = x[i]
            x[i] = keep + h
            up = np.sum(f(_NP(), *xs) * err)
            x[i] = keep - h
            dn = np.sum(f(_NP(), *xs) * err)
            x[i] = keep
            g[i] = (up - dn) / (2 * h)
        grads.append(g)
    return grads


def _backend_grads(be, f, arrays, err=None):
    tensors = [be.array(a) for a in arrays]
    tree = f(be, *tensors)
    ad = Autodiff(tree, be, next_error=None if err is None else be.array(err))
    return ad.get_grad_asnumpyarray(tensors)


def _hard_coded(be):
    """reference tests/test_autodiff.py test_hard_coded: x0..x3 constant 3x3
    tensors 1, 2, 3, 5"""
    xs = [be.array(np.full((3, 3), v, dtype=np.float32)) for v in (1, 2, 3, 5)]
    x0, x1, x2, x3 = xs
    f = x0 * x0 - x1 * x0 + x0 * x2 - x2 * x1 * x0 + x3 * x3 * x3
    got = Autodiff(f, be).get_grad_asnumpyarray(xs)
    for g, want in zip(got, (-3.0, -4.0, -1.0, 75.0)):
        assert_close(g, np.full((3, 3), want, dtype=np.float32), rtol=0, atol=1e-5)


def test_hard_coded_oracle(cpu):
    _hard_coded(cpu)


@pytest.mark.parametrize("name,f,shapes,kind", FUNCS, ids=IDS)
def test_numerical_gradient_oracle(cpu, name, f, shapes, kind):
    arrays = _inputs(shapes, kind, 7)
    out_shape = np.asarray(f(_NP(), *[a.astype(np.float64) for a in arrays])).shape
    err = np.random.RandomState(3).rand(*out_shape).astype(np.float32) + 0.5
    want = _numerical(f, arrays, err.astype(np.float64))
    got = _backend_grads(cpu, f, arrays, err)
    for i, (g, w) in enumerate(zip(got, want)):
        assert_close(g, w, rtol=2e-3, atol=2e-3 * max(1.0, np.abs(w).max()), what="%s d/dx%d" % (name, i))


def test_default_error_is_ones_and_unused_tensor_gets_zero(cpu):
    a, b = [cpu.array(x) for x in _inputs([(4, 5)] * 2, "rand", 1)]
    ad = Autodiff(a * 3.0, cpu)
    ga, gb = ad.get_grad_asnumpyarray([a, b])
    assert_close(ga, np.full((4, 5), 3.0, dtype=np.float32))
    assert_close(gb, np.zeros((4, 5), dtype=np.float32))


def test_comparisons_block_gradients(cpu):
    a, b = [cpu.array(x) for x in _inputs([(4, 5)] * 2, "rand", 2)]
    ga, gb = Autodiff((a > b) * a + cpu.sgn(b), cpu).get_grad_asnumpyarray([a, b])
    assert_close(ga, (a.get() > b.get()).astype(np.float32))
    assert_close(gb, np.zeros((4, 5), dtype=np.float32))


def test_back_prop_grad_writes_buffers_and_may_reuse_next_error(cpu):
    xa, xb = _inputs([(6, 4)] * 2, "rand", 5)
    a, b = cpu.array(xa), cpu.array(xb)
    err_np = np.random.RandomState(9).rand(6, 4).astype(np.float32)
    err = cpu.array(err_np)
    ga = cpu.empty((6, 4))
    ad = Autodiff(a * b + a, cpu, next_error=err)
    ad.back_prop_grad([a, b], [ga, err])
    assert_close(ga.get(), err_np * (xb + 1.0))
    assert_close(err.get(), err_np * xa)
    with pytest.raises(AssertionError):
        ad.back_prop_grad([a], [b])
    ad.cleanup()
    assert ad.map_tensor_grad_op_tree == {}


def test_next_error_shape_is_checked(cpu):
    a = cpu.array(np.ones((3, 4), dtype=np.float32))
    with pytest.raises(AssertionError):
        Autodiff(a * 2.0, cpu, next_error=cpu.ones((4, 3)))


def test_views_accumulate_on_their_base(cpu):
    x = _inputs([(6, 4)], "rand", 11)[0]
    a = cpu.array(x)
    g = Autodiff(a * a.reshape((6, 4)), cpu).get_grad_asnumpyarray([a])[0]
    assert_close(g, 2 * x)


# ---- GPU: the hip backend's gradients against the oracle's ---------------------------------

@pytest.mark.gpu
def test_hard_coded_hip(hip):
    _hard_coded(hip)


@pytest.mark.gpu
@pytest.mark.parametrize("name,f,shapes,kind", FUNCS, ids=IDS)
def test_gradients_hip_match_oracle(pair, name, f, shapes, kind):
    cpu, hip = pair
    big = [(s[0] * 31 if s[0] > 1 else 1, s[1] * 31 if s[1] > 1 else 1) for s in shapes]
    arrays = _inputs(big, kind, 13)
    out_shape = np.asarray(f(_NP(), *arrays)).shape
    err = np.random.RandomState(4).rand(*out_shape).astype(np.float32) + 0.5
    want = _backend_grads(cpu, f, arrays, err)
    got = _backend_grads(hip, f, arrays, err)
    for i, (g, w) in enumerate(zip(got, want)):
        # gradients that pass through sums over hundreds of terms: scale the
        # absolute floor with the magnitude of the result
        assert_close(g, w, rtol=1e-4, atol=1e-5 * max(1.0, np.abs(w).max()), what="%s d/dx%d" % (name, i))


@pytest.mark.gpu
def test_batchnorm_tree_hip(pair):
    """reference tests/test_autodiff.py test_batchnorm: normalise over axis 1,
    scale and shift, gradients for all three operands with an incoming error
    written back into the error buffer"""
    cpu, hip = pair
    rs = np.random.RandomState(21)
    x = rs.randn(64, 128).astype(np.float32)
    gamma = rs.rand(64, 1).astype(np.float32) + 0.5
    beta = rs.randn(64, 1).astype(np.float32)
    err_np = rs.randn(64, 128).astype(np.float32)
    results = []
    for be in (cpu, hip):
        x0, x1, x2 = be.array(x), be.array(gamma), be.array(beta)
        err = be.array(err_np)
        f = ((x0 - be.mean(x0, axis=1)) / be.sqrt(be.var(x0, axis=1) + 1e-6)) * x1 + x2
        g1, g2 = be.empty((64, 1)), be.empty((64, 1))
        Autodiff(f, be, next_error=err).back_prop_grad([x0, x1, x2], [err, g1, g2])
        results.append([err.get(), g1.get(), g2.get()])
    for g, w, what in zip(results[1], results[0], ("dx", "dgamma", "dbeta")):
        assert_close(g, w, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(w).max()), what=what)
    # closed form: dbeta = row sums of the error
    assert_close(results[1][2], err_np.astype(np.float64).sum(axis=1, keepdims=True).astype(np.float32),
                 rtol=1e-4, atol=1e-4)
