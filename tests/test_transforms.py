"""Activations, costs and metrics (neon_amd/transforms): the known answers the
reference's own tests hold (tests/test_activations.py, tests/test_costs.py) on
the oracle backend, then the hip backend against the oracle at sizes where the
reductions run as column kernels."""
import contextlib

import numpy as np
import pytest

from neon_amd import NervanaObject
from neon_amd.transforms import (Accuracy, CrossEntropyBinary, CrossEntropyMulti, Explin, GANCost, Identity,
                                 LogLoss, Logistic, MeanSquared, Misclassification, MultiMetric, Normalizer,
                                 PixelwiseSoftmax, PrecisionRecall, Rectlin, Rectlinclip, SmoothL1Loss, Softmax,
                                 SquareHingeLoss, SumSquared, Tanh, TopKMisclassification)
from utils import assert_close


@contextlib.contextmanager
def using(be, bsz=None):
    """make `be` the process-wide backend, as gen_backend would"""
    old, old_bsz = NervanaObject.be, be.bsz
    NervanaObject.be = be
    if bsz is not None:
        be.bsz = bsz
    try:
        yield be
    finally:
        NervanaObject.be, be.bsz = old, old_bsz


def _eval(be, tree, shape):
    if isinstance(tree, (int, float)):
        return np.full((1, 1), tree, dtype=np.float32)
    out = be.empty(shape)
    out[:] = tree
    return out.get()


def _act(be, func, inputs, deriv=False):
    x = be.array(np.asarray(inputs, dtype=np.float32))
    with using(be):
        tree = func.bprop(x) if deriv else func(x)
        return _eval(be, tree, np.asarray(inputs).shape)


def _cost(be, func, y, t, deriv=False):
    yt, tt = be.array(np.asarray(y, dtype=np.float32)), be.array(np.asarray(t, dtype=np.float32))
    with using(be):
        tree = func.bprop(yt, tt) if deriv else func(yt, tt)
        return _eval(be, tree, tree.shape)


col = lambda *v: np.array(v, dtype=np.float64).reshape((-1, 1))
EPS = np.exp(-50)

ACT_CASES = [
    # (name, transform, inputs, expected, derivative?, tolerance)  -- reference tests/test_activations.py
    ("identity", lambda: Identity(), col(0, 1, -2), col(0, 1, -2), False, 0),
    ("identity_d", lambda: Identity(), col(0, 1, -2), np.ones((1, 1)), True, 0),
    ("rectlin_pos", lambda: Rectlin(), col(1, 3, 2), col(1, 3, 2), False, 0),
    ("rectlin_neg", lambda: Rectlin(), [[-1, -3], [-2, -4]], [[0, 0], [0, 0]], False, 0),
    ("rectlin_mixed", lambda: Rectlin(), [[4, 0], [-2, 9]], [[4, 0], [0, 9]], False, 0),
    ("rectlin_d_pos", lambda: Rectlin(), col(1, 3, 2), col(1, 1, 1), True, 0),
    ("rectlin_d_neg", lambda: Rectlin(), [[-1, -3], [-2, -4]], [[0, 0], [0, 0]], True, 0),
    ("rectlin_d_mixed", lambda: Rectlin(), [[4, 0], [-2, 9]], [[1, 0], [0, 1]], True, 0),
    ("leaky_neg", lambda: Rectlin(slope=0.2), [[-1, -3], [-2, -4]], np.array([[-1, -3], [-2, -4]]) * 0.2, False, 1e-7),
    ("leaky_mixed", lambda: Rectlin(slope=0.2), [[4, 0], [-2, 9]], [[4, 0], [-0.4, 9]], False, 1e-7),
    ("leaky_d_mixed", lambda: Rectlin(slope=0.2), [[4, 0], [-2, 9]], [[1, 0], [0.2, 1]], True, 1e-7),
    ("softmax", lambda: Softmax(), col(0, 1, -2), np.exp(col(0, 1, -2) - 1) / np.sum(np.exp(col(0, 1, -2) - 1)), False, 1e-7),
    ("softmax_d", lambda: Softmax(), col(0, 1, -2), np.ones((1, 1)), True, 0),
    ("tanh", lambda: Tanh(), col(0, 1, -2), np.tanh(col(0, 1, -2)), False, 1e-7),
    ("tanh_d", lambda: Tanh(), np.tanh(col(0, 1, -2)), 1 - np.tanh(col(0, 1, -2)) ** 2, True, 1e-7),
    ("logistic", lambda: Logistic(), col(0, 1, -2), 1 / (1 + np.exp(-col(0, 1, -2))), False, 1e-7),
    ("logistic_d", lambda: Logistic(shortcut=False), 1 / (1 + np.exp(-col(0, 1, -2))),
     (1 / (1 + np.exp(-col(0, 1, -2)))) * (1 - 1 / (1 + np.exp(-col(0, 1, -2)))), True, 1e-7),
    ("logistic_shortcut", lambda: Logistic(shortcut=True), col(0.5, 0.7), np.ones((1, 1)), True, 0),
    # closed forms for the ones the reference's tests do not cover
    ("explin", lambda: Explin(alpha=0.5), col(2, 0, -1), col(2, 0, 0.5 * (np.exp(-1) - 1)), False, 1e-7),
    ("explin_d", lambda: Explin(alpha=0.5), col(2, -0.25), col(1, -0.25 + 0.5), True, 1e-7),
    ("rectlinclip", lambda: Rectlinclip(slope=0.1, xcut=3.0), col(5, 2, -2), col(3, 2, -0.2), False, 1e-7),
    ("rectlinclip_d", lambda: Rectlinclip(slope=0.1, xcut=3.0), col(5, 2, -2), col(0, 1, 0.1), True, 1e-7),
    ("normalizer", lambda: Normalizer(divisor=4.0), col(2, -8), col(0.5, -2), False, 0),
]


@pytest.mark.parametrize("name,make,inputs,expected,deriv,tol", ACT_CASES, ids=[c[0] for c in ACT_CASES])
def test_activation_known_answers(cpu, name, make, inputs, expected, deriv, tol):
    got = _act(cpu, make(), inputs, deriv)
    want = np.asarray(expected, dtype=np.float64)
    assert got.shape == want.shape or want.shape == (1, 1)
    assert np.all(np.abs(got - want) <= tol + 1e-12), (got, want)


def _pixelwise(be, c, x):
    with using(be):
        t = be.array(x)
        act = PixelwiseSoftmax(c=c)
        assert act(t) is t and act.bprop(t) == 1
        return t.get()


def test_pixelwise_softmax_known_answer(cpu):
    """reference tests/test_activations.py:187-201: two channels, three pixels, one image"""
    inputs = np.array([0, 1, 3, 1, 2, -2], dtype=np.float64).reshape((2, 3))
    e = np.exp(inputs - inputs.max(axis=0))
    got = _pixelwise(cpu, 2, inputs.reshape((1, -1)).astype(np.float32))
    assert np.all(np.abs(got - (e / e.sum(axis=0)).reshape((1, -1))) <= 1e-6)


def _pixelwise_case():
    rs = np.random.RandomState(31)
    c, pixels, batch = 21, 36 * 36, 8
    x = (rs.standard_normal((c * pixels, batch)) * 4).astype(np.float32)
    x64 = x.astype(np.float64).reshape(c, -1)
    e = np.exp(x64 - x64.max(axis=0))
    return c, x, (e / e.sum(axis=0)).reshape(x.shape)


def test_pixelwise_softmax_over_many_pixels(cpu):
    c, x, want = _pixelwise_case()
    assert_close(_pixelwise(cpu, c, x), want, rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_pixelwise_softmax_hip(pair):
    c, x, want = _pixelwise_case()
    got = [_pixelwise(be, c, x) for be in pair]
    assert_close(got[1], want, rtol=1e-5, atol=1e-7)
    assert_close(got[1], got[0], rtol=1e-5, atol=1e-7)


def _gan(be, func, y_data, y_noise):
    with using(be, bsz=y_data.shape[1]):
        cost = GANCost(func=func)
        yd, yn = be.array(y_data), be.array(y_noise)
        res = {}
        for kind in ("dis", "dis_data", "dis_noise", "gen"):
            out = be.iobuf(1)
            out[:] = cost(yd, yn, cost_type=kind)
            res[kind] = out.get()
        for name, fn, arg in (("d_data", cost.bprop_data, yd), ("d_noise", cost.bprop_noise, yn),
                              ("d_gen", cost.bprop_generator, yn)):
            delta = be.iobuf(y_data.shape[0])
            delta[:] = fn(arg)
            res[name] = delta.get()
        assert cost(yd, yn, cost_type="other") is None
        return res


def _gan_expected(func, yd, yn):
    """closed forms; each derivative is the derivative of the matching cost term
    (for 'modified' the reference keeps -1/y for the generator, the gradient
    of the 'original' generator cost: the usual non-saturating trick)"""
    yd, yn = yd.astype(np.float64), yn.astype(np.float64)
    slog = lambda v: np.log(np.maximum(v, np.exp(-50)))
    m = lambda v: v.mean(axis=0, keepdims=True)
    one = np.ones_like(yd)
    if func == "wasserstein":
        return {"dis": m(yd - yn), "dis_data": m(yd), "dis_noise": m(-yn), "gen": m(yn),
                "d_data": one, "d_noise": -one, "d_gen": one}
    gen = -slog(yn) if func == "original" else slog(1 - yn)
    return {"dis": m(-slog(yd) - slog(1 - yn)), "dis_data": m(-slog(yd)), "dis_noise": m(-slog(1 - yn)),
            "gen": m(gen), "d_data": -1 / yd, "d_noise": 1 / (1 - yn),
            "d_gen": 1 / (yn - 1) if func == "original" else -1 / yn}


def _gan_inputs(rows=5, batch=7):
    rs = np.random.RandomState(41)
    return (rs.uniform(0.05, 0.95, (rows, batch)).astype(np.float32),
            rs.uniform(0.05, 0.95, (rows, batch)).astype(np.float32))


@pytest.mark.parametrize("func", ["original", "modified", "wasserstein"])
def test_gan_cost_closed_forms(cpu, func):
    yd, yn = _gan_inputs()
    got, want = _gan(cpu, func, yd, yn), _gan_expected(func, yd, yn)
    for k in want:
        assert_close(got[k], want[k], rtol=2e-6, atol=1e-6, what=k)
    # the reference's own case (tests/test_gan.py:49-76): y_data = 1, y_noise = 2, where 1 - y_noise is clamped
    ones, twos = np.ones((5, 7), np.float32), np.full((5, 7), 2, np.float32)
    got = _gan(cpu, func, ones, twos)
    if func == "modified":
        assert np.all(got["dis"] == 50.0) and np.all(got["d_data"] == -1) and np.all(got["d_noise"] == -1)
        assert np.all(got["d_gen"] == -0.5)
    if func == "wasserstein":
        assert np.all(got["dis"] == -1.0) and np.all(got["d_gen"] == 1)
    with using(cpu, bsz=4):
        with pytest.raises(AssertionError):
            GANCost(func="other")
        with pytest.raises(AssertionError):
            GANCost(cost_type="both")


@pytest.mark.gpu
@pytest.mark.parametrize("func", ["original", "modified", "wasserstein"])
def test_gan_cost_hip(pair, func):
    yd, yn = _gan_inputs(rows=300, batch=512)
    res = [_gan(be, func, yd, yn) for be in pair]
    want = _gan_expected(func, yd, yn)
    for k in want:
        assert_close(res[1][k], want[k], rtol=2e-5, atol=1e-6, what=k)
        assert_close(res[1][k], res[0][k], rtol=2e-5, atol=1e-6, what=k)


def test_multi_metric_picks_one_output(cpu):
    rs = np.random.RandomState(3)
    with using(cpu, bsz=6):
        outs = tuple(cpu.array(rs.uniform(0.1, 1, (4, 6)).astype(np.float32)) for _ in range(3))
        mm = MultiMetric(LogLoss(), 1)
        assert mm.metric_names == ['LogLoss']                      # attributes come from the wrapped metric
        y = outs[1].get().astype(np.float64)
        assert abs(float(mm(outs, None)) - np.mean(-np.log((y * y).sum(axis=0)))) < 1e-6


def test_softmax_big_inputs(cpu):
    """reference tests/test_activations.py:156-184: 1000 classes, large logits"""
    rs = np.random.RandomState(1)
    x = rs.random_sample((1000, 128)) * 100
    got = _act(cpu, Softmax(), x)
    m = x.max(axis=0, keepdims=True)
    want = np.exp(x - m) / np.exp(x - m).sum(axis=0, keepdims=True)
    assert_close(got, want.astype(np.float32), rtol=1e-5, atol=1e-7)


Y1, T1 = col(0.5, 0.9, 0.1, 0.0001), col(0.5, 0.99, 0.01, 0.2)
Y2, T2 = col(0.5, 1.0, 0.0, 0.0001), col(0.5, 0.0, 1.0, 0.2)


def _ceb(y, t):
    return np.sum(-t * np.log(np.maximum(y, EPS)) - (1 - t) * np.log(np.maximum(1 - y, EPS)), keepdims=True)


def _cem(y, t):
    return np.sum(-t * np.log(np.maximum(y, EPS)), axis=0, keepdims=True)


COST_CASES = [
    # reference tests/test_costs.py:66-184
    ("ce_binary", lambda: CrossEntropyBinary(), Y1, T1, _ceb(Y1, T1), False, 1e-6),
    ("ce_binary_limits", lambda: CrossEntropyBinary(), Y2, T2, _ceb(Y2, T2), False, 1e-5),
    ("ce_binary_d", lambda: CrossEntropyBinary(), Y2, T2, (Y2 - T2), True, 1e-6),
    ("ce_multi", lambda: CrossEntropyMulti(), Y1, T1, _cem(Y1, T1), False, 1e-6),
    ("ce_multi_limits", lambda: CrossEntropyMulti(), Y2, T2, _cem(Y2, T2), False, 1e-5),
    ("ce_multi_d", lambda: CrossEntropyMulti(), Y2, T2, (Y2 - T2), True, 1e-6),
    ("ce_multi_bits", lambda: CrossEntropyMulti(usebits=True), Y1, T1, _cem(Y1, T1) / np.log(2), False, 1e-6),
    ("sum_squared", lambda: SumSquared(), Y1, T1, np.sum((Y1 - T1) ** 2, axis=0, keepdims=True) / 2, False, 1e-7),
    ("sum_squared_d", lambda: SumSquared(), Y2, T2, (Y2 - T2), True, 1e-7),
    ("mean_squared", lambda: MeanSquared(), Y1, T1, np.mean((Y1 - T1) ** 2, axis=0, keepdims=True) / 2, False, 1e-7),
    ("mean_squared_d", lambda: MeanSquared(), Y2, T2, (Y2 - T2) / 4, True, 1e-7),
    ("hinge", lambda: SquareHingeLoss(), col(0.5, -2, 3), col(1, -1, -1),
     np.mean(np.maximum(1 - col(1, -1, -1) * col(0.5, -2, 3), 0) ** 2, axis=0, keepdims=True), False, 1e-6),
]


@pytest.mark.parametrize("name,make,y,t,expected,deriv,tol", COST_CASES, ids=[c[0] for c in COST_CASES])
def test_cost_known_answers(cpu, name, make, y, t, expected, deriv, tol):
    got = _cost(cpu, make(), y, t, deriv)
    assert got.shape == np.asarray(expected).shape
    assert np.all(np.abs(got - expected) <= tol), (got, expected)


@pytest.mark.parametrize("sigma", [1.0, 0.5, 2.0])
@pytest.mark.parametrize("magnitude", [0.1, 10.0])
def test_smooth_l1(cpu, sigma, magnitude):
    """reference tests/test_costs.py:243-300 (value and derivative)"""
    rs = np.random.RandomState(3)
    y, t = (rs.random_sample((7, 5)) - 0.5) * magnitude, rs.random_sample((7, 5))
    x, s2 = y - t, sigma ** 2
    small = np.abs(x) < 1.0 / s2
    want = np.where(small, 0.5 * x ** 2 * s2, np.abs(x) - 0.5 / s2).sum(axis=0, keepdims=True)
    assert_close(_cost(cpu, SmoothL1Loss(sigma=sigma), y, t), want.astype(np.float32), rtol=1e-5, atol=1e-6)
    dwant = np.where(small, x * s2, np.sign(x))
    assert_close(_cost(cpu, SmoothL1Loss(sigma=sigma), y, t, deriv=True), dwant.astype(np.float32), rtol=1e-5, atol=1e-6)


def test_cross_entropy_shape_check(cpu):
    with using(cpu):
        with pytest.raises(ValueError):
            CrossEntropyMulti()(cpu.zeros((4, 2)), cpu.zeros((4, 3)))


def _metrics(be):
    """the reference's metric known answers (tests/test_costs.py:200-235) plus
    log loss / accuracy / top-k on the same small case"""
    out = {}
    y = np.array([[0.25, 0.99, 0.33], [0.5, 0.005, 0.32], [0.25, 0.005, 0.34]], dtype=np.float32)
    t = np.array([[0, 1, 0], [1, 0, 1], [0, 0, 0]], dtype=np.float32)
    with using(be, bsz=3):
        out["mis"] = Misclassification()(be.array(y), be.array(t))
        out["acc"] = Accuracy()(be.array(y), be.array(t))
        out["logloss"] = LogLoss()(be.array(y), be.array(t))
        out["top2"] = TopKMisclassification(2)(be.array(y), be.array(t))
    preds = np.array([[0, 1, 0, 1], [1, 0, 0, 0], [0, 0, 1, 0]], dtype=np.float32)
    soft = np.array([[0.2, 0.9, 0.01, 1], [0.75, 0.05, 0.44, 0], [0.05, 0.05, 0.55, 0]], dtype=np.float32)
    targ = np.array([[0, 1, 0, 1], [1, 0, 1, 0], [0, 0, 0, 0]], dtype=np.float32)
    with using(be, bsz=4):
        out["pr"] = PrecisionRecall(3)(be.array(preds), be.array(targ))
        out["pr_bin"] = PrecisionRecall(3, binarize=True)(be.array(soft), be.array(targ))
    return out


def _check_metrics(m):
    assert abs(m["mis"] - 1.0 / 3) < 1e-7
    assert abs(m["acc"] - 2.0 / 3) < 1e-7
    assert abs(float(m["logloss"]) - (-np.log([0.5, 0.99, 0.32]).mean())) < 1e-6
    assert_close(m["pr"], np.array([2, 1.5]) / 3, rtol=1e-5, atol=1e-6)
    assert_close(m["pr_bin"], np.array([2, 1.5]) / 3, rtol=1e-5, atol=1e-6)
    # sample 3: the true class (0.32) is the third largest of (0.33, 0.32, 0.34): a top-2 miss
    assert_close(m["top2"], np.array([-np.log([0.5, 0.99, 0.32]).mean(), 1.0 / 3, 1.0 / 3]), rtol=1e-5, atol=1e-6)


def test_metric_known_answers(cpu):
    _check_metrics(_metrics(cpu))


# ---- GPU --------------------------------------------------------------------------------
@pytest.mark.gpu
def test_metric_known_answers_hip(hip):
    _check_metrics(_metrics(hip))


@pytest.mark.gpu
@pytest.mark.parametrize("name,make", [
    ("rectlin", lambda: Rectlin(slope=0.1)), ("rectlinclip", lambda: Rectlinclip(slope=0.1, xcut=1.5)),
    ("explin", lambda: Explin(alpha=0.7)), ("tanh", lambda: Tanh()), ("logistic", lambda: Logistic()),
    ("softmax0", lambda: Softmax()), ("softmax1", lambda: Softmax(axis=1)), ("normalizer", lambda: Normalizer(divisor=3.0)),
])
def test_activations_hip_match_oracle(pair, name, make):
    x = (np.random.RandomState(8).standard_normal((1000, 384)) * 2).astype(np.float32)
    for deriv in (False, True):
        got = [_act(be, make(), x, deriv) for be in pair]
        assert_close(got[1], got[0], rtol=1e-5, atol=1e-6, what="%s deriv=%s" % (name, deriv))


@pytest.mark.gpu
@pytest.mark.parametrize("name,make", [
    ("ce_binary", lambda: CrossEntropyBinary()), ("ce_multi", lambda: CrossEntropyMulti()),
    ("ce_multi_bits", lambda: CrossEntropyMulti(usebits=True, scale=0.5)), ("sum_squared", lambda: SumSquared()),
    ("mean_squared", lambda: MeanSquared()), ("smooth_l1", lambda: SmoothL1Loss(sigma=1.5)),
    ("hinge", lambda: SquareHingeLoss(margin=0.8)),
])
def test_costs_hip_match_oracle(pair, name, make):
    rs = np.random.RandomState(9)
    logits = rs.standard_normal((1000, 256)) * 3
    y = np.exp(logits - logits.max(axis=0)) / np.exp(logits - logits.max(axis=0)).sum(axis=0)
    t = np.zeros_like(y)
    t[rs.randint(0, 1000, size=256), np.arange(256)] = 1
    y[0, :4] = 0.0                                                    # exercises the clamp of safelog
    for deriv in (False, True):
        got = [_cost(be, make(), y, t, deriv) for be in pair]
        # sums over 1000 classes: absolute floor scaled by the magnitude of the result
        assert_close(got[1], got[0], rtol=2e-5, atol=1e-6 * max(1.0, np.abs(got[0]).max()),
                     what="%s deriv=%s" % (name, deriv))


@pytest.mark.gpu
def test_classification_metrics_hip_match_oracle(pair):
    rs = np.random.RandomState(10)
    nclass, batch = 1000, 512
    logits = rs.standard_normal((nclass, batch)) * 2
    y = (np.exp(logits) / np.exp(logits).sum(axis=0)).astype(np.float32)
    labels = np.where(rs.rand(batch) < 0.5, y.argmax(axis=0), rs.randint(0, nclass, size=batch))
    t = np.zeros_like(y)
    t[labels, np.arange(batch)] = 1
    res = []
    for be in pair:
        with using(be, bsz=batch):
            yt, tt = be.array(y), be.array(t)
            res.append((Misclassification()(yt, tt), Accuracy()(yt, tt), float(LogLoss()(yt, tt)),
                        TopKMisclassification(5)(yt, tt), PrecisionRecall(nclass, binarize=True)(be.array(y), tt)))
    assert res[1][0] == res[0][0] == np.float32((y.argmax(axis=0) != labels).mean())
    assert res[1][1] == res[0][1]
    assert abs(res[1][2] - res[0][2]) < 1e-5
    assert_close(res[1][3], res[0][3], rtol=1e-5, atol=1e-6)
    assert_close(res[1][4], res[0][4], rtol=1e-5, atol=1e-6)


# ---- layer-facing helpers of the Backend base ---------------------------------------
class _Branch(object):
    """stands in for a layer: y (+)= w * x going forward, deltas (+)= alpha * w * error back"""

    def __init__(self, be, w, out, deltas):
        self.be, self.w, self.out, self.deltas = be, w, out, deltas

    def fprop(self, inputs, inference, beta=0):
        self.out[:] = self.out * beta + inputs * self.w

    def bprop(self, error, alpha=1.0, beta=0.0):
        self.deltas[:] = self.deltas * beta + error * (alpha * self.w)


def test_merge_helpers_drive_branches_with_the_right_accumulation(cpu):
    be = cpu
    x = be.array(np.arange(6, dtype=np.float32).reshape(2, 3))
    out, deltas = be.array(np.full((2, 3), 100.0, np.float32)), be.array(np.full((2, 3), 10.0, np.float32))
    branches = [_Branch(be, w, out, deltas) for w in (1.0, 2.0, 4.0)]
    assert be.relu_layer() is None and be.batchnorm_layer((3, 4, 4)) is None
    assert be.mergesum_layer(3) is None and be.mergebroadcast_layer(3) is None
    be.fprop_mergesum(None, x, False, branches, out, None)
    assert np.array_equal(out.get(), 7.0 * x.get())             # the stale 100s are overwritten
    be.bprop_mergesum(None, 0.5, 2.0, branches, x, deltas)
    assert np.array_equal(deltas.get(), 2.0 * 10.0 + 0.5 * 7.0 * x.get())
    # broadcast merge: every branch has its own error view and its own (alpha, beta)
    d = [be.array(np.full((2, 3), 1.0, np.float32)) for _ in range(3)]
    outs = [be.zeros((2, 3)) for _ in range(3)]
    bb = [_Branch(be, w, o, dk) for w, o, dk in zip((1.0, 2.0, 4.0), outs, d)]
    be.fprop_mergebroadcast(None, x, False, None, bb, None)
    assert all(np.array_equal(o.get(), w * x.get()) for o, w in zip(outs, (1.0, 2.0, 4.0)))
    betas = [1.0, 0.0, None]
    be.bprop_mergebroadcast(None, bb, [x, x, x], x, None, None, 2.0, 3.0, [1.0, 0.5, 0.25], betas)
    assert betas[-1] == 3.0
    want = [1.0 + 2.0 * x.get(), 0.0 + 2.0 * x.get(), 3.0 + 2.0 * x.get()]
    assert all(np.array_equal(dk.get(), w) for dk, w in zip(d, want))


def test_small_aliases_of_the_backend_base(cpu):
    be = cpu
    x = be.array(np.array([[1.0, -2.0, 4.0], [-8.0, 16.0, -32.0]], np.float32))
    out = be.empty((2, 3))
    be.fabs(x, out=out)
    assert np.array_equal(out.get(), np.abs(x.get()))
    be.true_divide(x, 2.0, out=out)
    assert np.array_equal(out.get(), x.get() / 2)
    bias = be.array(np.array([[10.0], [20.0]], np.float32))
    grad = be.empty((2, 1))
    be.update_fc_bias(x, grad)
    assert np.array_equal(grad.get(), x.get().sum(axis=1, keepdims=True))
    be.add_fc_bias(x, bias)
    assert np.array_equal(x.get(), np.array([[11.0, 8.0, 14.0], [12.0, 36.0, -12.0]], np.float32))
    assert be.is_mkl() is False and be.convert_data(x, False) is None and be.clean_data(x, False) is None
    assert be.allocate_new_deltas(x, (2, 3), "Data") is x
