"""Parameter update rules (neon_amd/optimizers): each rule against a float64
numpy restatement of its formula -- the reference's own test idiom
(tests/test_optimizer.py:73-300) -- on the oracle backend, then the hip backend
against the oracle over several steps, and the fusion of every update into one
kernel."""
import numpy as np
import pytest

from neon_amd.optimizers import (Adadelta, Adagrad, Adam, ExpSchedule, GradientDescentMomentum,
                                 MultiOptimizer, PolySchedule, PowerSchedule, RMSProp, Schedule,
                                 StepSchedule)
from utils import assert_close

SHAPE = (200, 128)
BSZ = 128


class DummyLayer(object):
    def __init__(self, plist, name=None):
        self.plist, self.name = plist, name

    def get_params(self):
        return self.plist


def _setup(be, n_states, seed=0, shape=SHAPE, nparams=1):
    rs = np.random.RandomState(seed)
    host, plist = [], []
    for _ in range(nparams):
        p, g = rs.rand(*shape), 0.01 * rs.rand(*shape)
        st = [0.01 * rs.rand(*shape) for _ in range(n_states)]
        host.append((p, g, st))
        plist.append(((be.array(p.astype(np.float32)), be.array(g.astype(np.float32))),
                      [be.array(s.astype(np.float32)) for s in st]))
    return host, plist


def _run(opt, be, plist, epoch=1):
    opt.be = be
    old = be.bsz
    be.bsz = BSZ
    try:
        opt.optimize([DummyLayer(plist)], epoch=epoch)
    finally:
        be.bsz = old


# ---- float64 restatements --------------------------------------------------------------
def np_gdm(p, g, st, lr, mom, wd, nesterov=False, clip=None, scale=1.0):
    g = scale * g / BSZ + wd * p
    v = mom * st[0] - lr * g
    p = p + mom * v - lr * g if nesterov else p + v
    if clip:
        p = np.clip(p, -clip, clip)
    return p, [v]


def np_rmsprop(p, g, st, lr, decay, eps, clip=None):
    g = g / BSZ
    if clip:
        g = np.clip(g, -clip, clip)
    s = decay * st[0] + g * g * (1 - decay)
    return p - g * lr / (np.sqrt(s + eps) + eps), [s]


def np_adagrad(p, g, st, lr, eps):
    g = g / BSZ
    s = st[0] + g * g
    return p - g * lr / np.sqrt(s + eps), [s]


def np_adadelta(p, g, st, decay, eps):
    g = g / BSZ
    gsq = st[0] * decay + (1 - decay) * g * g
    upd = np.sqrt((st[1] + eps) / (gsq + eps)) * g
    usq = st[1] * decay + (1 - decay) * upd * upd
    return p - upd, [gsq, usq, upd]


def np_adam(p, g, st, lr, b1, b2, eps, t):
    g = g / BSZ
    m = st[0] * b1 + (1 - b1) * g
    v = st[1] * b2 + (1 - b2) * g * g
    step = lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t)
    return p - step * m / (np.sqrt(v) + eps), [m, v]


CASES = [
    ("gdm", lambda: GradientDescentMomentum(0.1, 0.9, wdecay=0.005), 1,
     lambda p, g, st, t: np_gdm(p, g, st, 0.1, 0.9, 0.005)),
    ("gdm_wclip", lambda: GradientDescentMomentum(0.1, 0.9, wdecay=0.005, param_clip_value=0.5), 1,
     lambda p, g, st, t: np_gdm(p, g, st, 0.1, 0.9, 0.005, clip=0.5)),
    ("gdm_nesterov", lambda: GradientDescentMomentum(0.1, 0.9, wdecay=0.005, nesterov=True), 1,
     lambda p, g, st, t: np_gdm(p, g, st, 0.1, 0.9, 0.005, nesterov=True)),
    ("rmsprop", lambda: RMSProp(decay_rate=0.95, learning_rate=2e-3, epsilon=1e-6), 1,
     lambda p, g, st, t: np_rmsprop(p, g, st, 2e-3, 0.95, 1e-6)),
    ("rmsprop_gclip", lambda: RMSProp(decay_rate=0.95, learning_rate=2e-3, epsilon=1e-6, gradient_clip_value=4e-5), 1,
     lambda p, g, st, t: np_rmsprop(p, g, st, 2e-3, 0.95, 1e-6, clip=4e-5)),
    ("adagrad", lambda: Adagrad(learning_rate=0.01, epsilon=1e-6), 1,
     lambda p, g, st, t: np_adagrad(p, g, st, 0.01, 1e-6)),
    ("adadelta", lambda: Adadelta(decay=0.95, epsilon=1e-6), 3,
     lambda p, g, st, t: np_adadelta(p, g, st, 0.95, 1e-6)),
    ("adam", lambda: Adam(learning_rate=0.001, beta_1=0.9, beta_2=0.999, epsilon=1e-8), 2,
     lambda p, g, st, t: np_adam(p, g, st, 0.001, 0.9, 0.999, 1e-8, t)),
]
IDS = [c[0] for c in CASES]


@pytest.mark.parametrize("name,make,n_states,ref", CASES, ids=IDS)
def test_rule_matches_numpy_on_the_oracle(cpu, name, make, n_states, ref):
    host, plist = _setup(cpu, n_states)
    opt = make()
    (p, g, st) = host[0]
    for t in (1, 2, 3):
        _run(opt, cpu, plist)
        p, st = ref(p, g, st, t)
        (param, grad), states = plist[0]
        assert_close(param.get(), p.astype(np.float32), rtol=2e-6, atol=1e-7, what="%s step %d" % (name, t))
        for s_dev, s_np in zip(states, st):
            assert_close(s_dev.get(), s_np.astype(np.float32), rtol=1e-5, atol=1e-9)


def test_states_are_created_on_first_use(cpu):
    rs = np.random.RandomState(1)
    plist = [((cpu.array(rs.rand(8, 4).astype(np.float32)), cpu.array(rs.rand(8, 4).astype(np.float32))), [])]
    _run(Adam(), cpu, plist)
    assert len(plist[0][1]) == 2 and plist[0][1][0].shape == (8, 4)
    plist2 = [((cpu.array(rs.rand(8, 4).astype(np.float32)), cpu.array(rs.rand(8, 4).astype(np.float32))), [])]
    _run(GradientDescentMomentum(0.1, 0), cpu, plist2)
    assert plist2[0][1] == []                      # no momentum: no velocity buffer


def test_gradient_norm_clipping(cpu):
    host, plist = _setup(cpu, 1, seed=3, nparams=2)
    opt = GradientDescentMomentum(0.1, 0.9, gradient_clip_norm=1e-4)
    norm = np.sqrt(sum((g ** 2).sum() for p, g, st in host)) / BSZ
    scale = 1e-4 / max(norm, 1e-4)
    assert scale < 1
    _run(opt, cpu, plist)
    for (p, g, st), ((param, grad), states) in zip(host, plist):
        want, _ = np_gdm(p, g, st, 0.1, 0.9, 0.0, scale=scale)
        assert_close(param.get(), want.astype(np.float32), rtol=2e-6, atol=1e-7)


def test_nesterov_needs_momentum():
    with pytest.raises(ValueError):
        GradientDescentMomentum(0.1, 0, nesterov=True)


def test_schedules():
    lr = 0.1
    s = Schedule()
    assert [s.get_learning_rate(lr, e) for e in range(3)] == [lr] * 3
    s = Schedule(step_config=[2, 4], change=0.5)
    assert np.allclose([s.get_learning_rate(lr, e) for e in range(6)], [.1, .1, .05, .05, .025, .025])
    s = Schedule(step_config=2, change=0.1)
    assert np.allclose([s.get_learning_rate(lr, e) for e in range(5)], [.1, .1, .01, .01, .001])
    s = StepSchedule([1, 3], [0.2, 0.05])
    assert [s.get_learning_rate(lr, e) for e in range(5)] == [lr, 0.2, 0.2, 0.05, 0.05]
    s = PowerSchedule(2, 0.5)
    assert np.allclose([s.get_learning_rate(lr, e) for e in range(5)], [.1, .1, .05, .05, .025])
    s = ExpSchedule(0.5)
    assert np.allclose([s.get_learning_rate(lr, e) for e in range(3)], [.1, .1 / 1.5, .05])
    s = PolySchedule(4, 2.0)
    assert np.allclose([s.get_learning_rate(lr, e) for e in (0, 3, 4)], [.1, .1, 0.0])
    with pytest.raises(AssertionError):
        StepSchedule([1, 2], [0.1])


def test_multi_optimizer_routes_layers(cpu):
    _, pa = _setup(cpu, 0, seed=5)
    _, pb = _setup(cpu, 0, seed=6)
    a0, b0 = pa[0][0][0].get().copy(), pb[0][0][0].get().copy()
    fast, slow = GradientDescentMomentum(1.0, 0), GradientDescentMomentum(0.0, 0)
    multi = MultiOptimizer({"default": slow, "special": fast})
    for o in (fast, slow, multi):
        o.be = cpu
    old, cpu.bsz = cpu.bsz, 1
    try:
        multi.optimize([DummyLayer(pa, name="special"), DummyLayer(pb, name="other")], epoch=0)
    finally:
        cpu.bsz = old
    assert not np.allclose(pa[0][0][0].get(), a0) and np.array_equal(pb[0][0][0].get(), b0)
    with pytest.raises(AssertionError):
        MultiOptimizer({"special": fast})


# ---- GPU --------------------------------------------------------------------------------
@pytest.mark.gpu
@pytest.mark.parametrize("name,make,n_states,ref", CASES, ids=IDS)
def test_rule_hip_matches_oracle_and_fuses(pair, name, make, n_states, ref):
    cpu, hip = pair
    shape = (300, 257)                                   # odd row length: unaligned tail paths
    _, pl_cpu = _setup(cpu, n_states, seed=11, shape=shape, nparams=2)
    _, pl_hip = _setup(hip, n_states, seed=11, shape=shape, nparams=2)
    o_cpu, o_hip = make(), make()
    for t in range(4):
        before = hip.plan_stats["launches"]
        _run(o_cpu, cpu, pl_cpu, epoch=t)
        _run(o_hip, hip, pl_hip, epoch=t)
        assert hip.plan_stats["launches"] - before == 2, "one kernel per parameter"
    for ((pc, _), sc), ((ph, _), sh) in zip(pl_cpu, pl_hip):
        assert_close(ph.get(), pc.get(), rtol=1e-5, atol=1e-7, what=name)
        for a, b in zip(sh, sc):
            assert_close(a.get(), b.get(), rtol=1e-5, atol=1e-9, what=name + " state")


@pytest.mark.gpu
def test_gradient_norm_clipping_hip(pair):
    cpu, hip = pair
    res = []
    for be in pair:
        _, plist = _setup(be, 1, seed=3, nparams=3)
        _run(RMSProp(gradient_clip_norm=5e-5, gradient_clip_value=1e-4, param_clip_value=0.9), be, plist)
        res.append([p.get() for (p, g), st in plist])
    for a, b in zip(res[1], res[0]):
        assert_close(a, b, rtol=1e-5, atol=1e-7)


@pytest.mark.gpu
def test_adam_stochastic_rounding_fp16_params(hip):
    """fp16 parameters with stochastic rounding keep learning where
    round-to-nearest stalls: 200 steps of a constant tiny gradient"""
    shape = (64, 128)
    res = {}
    for sr in (False, 10):
        p = hip.array(np.ones(shape, np.float16), dtype=np.float16)
        g = hip.array(np.full(shape, 1.0, np.float32))
        plist = [((p, g), [])]
        opt = GradientDescentMomentum(1e-4, 0, stochastic_round=sr)
        opt.be = hip
        old, hip.bsz = hip.bsz, 1
        try:
            for _ in range(200):
                opt.optimize([DummyLayer(plist)], epoch=0)
        finally:
            hip.bsz = old
        res[sr] = p.get().astype(np.float64).mean()
    assert res[False] == 1.0                              # 1e-4 is below half a unit in the last place of 1.0
    assert abs(res[10] - (1.0 - 200 * 1e-4)) < 2e-3
