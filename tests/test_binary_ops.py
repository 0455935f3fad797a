"""binarize / shift (the helpers of the reference's binary networks,
nervanacpu.py:1823-1863): closed forms on the oracle, hip against the oracle."""
import numpy as np
import pytest

from utils import assert_close


def _np_shift(a, s, value=True):
    if value:
        e = np.rint(np.log(np.maximum(np.abs(s), np.exp(-50.0))) / np.log(2.0))
        return a * np.sign(s) * np.exp2(e)
    return a * np.exp2(s)


def _sign_case(be):
    # reference tests/test_activations.py:248-251
    x = be.array(np.array([-1, -.5, 0, .5, 1], dtype=np.float32).reshape((5, 1)))
    be.binarize(x, x, stochastic=False)       # what the Sign activation does (activation.py:372-382)
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
