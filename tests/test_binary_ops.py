"""binarize / shift (the helpers of the reference's binary networks,
nervanacpu.py:1823-1863) and their callers Sign, ShiftSchedule, ShiftAdaMax:
closed forms on the oracle, hip against the oracle."""
import numpy as np
import pytest

from neon_amd.optimizers import ShiftAdaMax, ShiftSchedule
from neon_amd.transforms import Sign
from utils import assert_close


def _np_shift(a, s, value=True):
    if value:
        e = np.rint(np.log(np.maximum(np.abs(s), np.exp(-50.0))) / np.log(2.0))
        return a * np.sign(s) * np.exp2(e)
    return a * np.exp2(s)


def _sign_case(be):
    # reference tests/test_activations.py:248-251
    x = be.array(np.array([-1, -.5, 0, .5, 1], dtype=np.float32).reshape((5, 1)))
    act = Sign()
    act.be = be
    act(x)
    return x.get()


def _shift_cases(be, a, s):
    A, S = be.array(a), be.array(s)
    by_value = be.shift(A, S).get()
    by_exponent = be.shift(A, be.array(np.rint(s * 3)), value=False).get()
    scalar = be.shift(A, 0.3).get()
    return by_value, by_exponent, scalar


def test_sign_and_deterministic_binarize(cpu):
    assert np.array_equal(_sign_case(cpu), np.array([-1, -1, 1, 1, 1], dtype=np.float32).reshape((5, 1)))


def test_shift_closed_forms(cpu):
    rs = np.random.RandomState(0)
    a = rs.standard_normal((6, 7)).astype(np.float32)
    s = (rs.standard_normal((6, 7)) * 4).astype(np.float32)
    by_value, by_exponent, scalar = _shift_cases(cpu, a, s)
    assert_close(by_value, _np_shift(a, s).astype(np.float32), rtol=1e-6, atol=0)
    assert_close(by_exponent, _np_shift(a, np.rint(s * 3), value=False).astype(np.float32), rtol=1e-6, atol=0)
    assert_close(scalar, (a * 0.25).astype(np.float32), rtol=0, atol=0)       # 0.3 rounds to 2^-2


def test_stochastic_binarize_oracle(cpu):
    x = np.linspace(-1.5, 1.5, 7, dtype=np.float32).reshape((7, 1)) * np.ones((1, 4000), np.float32)
    out = cpu.empty(x.shape)
    cpu.binarize(cpu.array(x), out, stochastic=True)
    got = out.get()
    assert np.all((got == 1) | (got == -1))
    p_plus = (got == 1).mean(axis=1)
    assert_close(p_plus, np.clip((x[:, 0] + 1) / 2, 0, 1), rtol=0, atol=0.04)


def test_shift_schedule(cpu):
    s = ShiftSchedule(interval=2, shift_size=1)
    s.be = cpu
    assert [s.get_learning_rate(0.5, e) for e in range(5)] == [0.5, 0.5, 0.25, 0.25, 0.125]


def _adamax(be, steps=3):
    rs = np.random.RandomState(4)
    p = be.array(rs.uniform(-1, 1, (30, 17)).astype(np.float32))
    g = be.array((rs.standard_normal((30, 17)) * 0.1).astype(np.float32))
    opt = ShiftAdaMax(learning_rate=0.01)
    opt.be = be

    class L(object):
        plist = [((p, g), [])]

        def get_params(self):
            return self.plist

    old, be.bsz = be.bsz, 4
    try:
        for e in range(steps):
            opt.optimize([L()], epoch=e)
    finally:
        be.bsz = old
    return p.get(), [s.get() for s in L.plist[0][1]]


def test_shift_adamax_oracle_first_step(cpu):
    rs = np.random.RandomState(4)
    p0 = rs.uniform(-1, 1, (30, 17)).astype(np.float32)
    g0 = (rs.standard_normal((30, 17)) * 0.1).astype(np.float32)
    got, states = _adamax(cpu, steps=1)
    g = g0.astype(np.float64) / 4
    m = 0.1 * g
    v = np.abs(g)
    want = np.clip(p0 - _np_shift(_np_shift(m, 1.0 / (v + 1e-8)), 0.01 / (1 - 0.9)), -1, 1)
    assert_close(got, want.astype(np.float32), rtol=1e-5, atol=1e-6)


# ---- GPU --------------------------------------------------------------------------------
@pytest.mark.gpu
def test_binary_ops_hip(pair):
    cpu, hip = pair
    assert np.array_equal(_sign_case(hip), _sign_case(cpu))
    rs = np.random.RandomState(1)
    a = rs.standard_normal((130, 257)).astype(np.float32)
    s = (rs.standard_normal((130, 257)) * 4).astype(np.float32)
    for g, w in zip(_shift_cases(hip, a, s), _shift_cases(cpu, a, s)):
        assert_close(g, w, rtol=1e-6, atol=0)
    x = np.linspace(-1.5, 1.5, 7, dtype=np.float32).reshape((7, 1)) * np.ones((1, 8192), np.float32)
    out = hip.empty(x.shape)
    hip.binarize(hip.array(x), out, stochastic=True)
    got = out.get()
    assert np.all((got == 1) | (got == -1))
    assert_close((got == 1).mean(axis=1), np.clip((x[:, 0] + 1) / 2, 0, 1), rtol=0, atol=0.03)
    sched = ShiftSchedule(interval=3)
    sched.be = hip
    assert [sched.get_learning_rate(1.0, e) for e in (0, 3, 7)] == [1.0, 0.5, 0.25]


@pytest.mark.gpu
def test_shift_adamax_hip_matches_oracle(pair):
    (pc, sc), (ph, sh) = _adamax(pair[0]), _adamax(pair[1])
    assert_close(ph, pc, rtol=1e-5, atol=1e-6)
    for a, b in zip(sh, sc):
        assert_close(a, b, rtol=1e-5, atol=1e-9)
