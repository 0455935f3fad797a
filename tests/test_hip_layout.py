"""Layout and accumulation helpers next to the op-tree path: copy_transpose
(dimension shuffle) and compensated_sum (Kahan accumulation into low-precision
storage).  Bit-exact bars: a shuffle moves values unchanged; the compensated
update is a fixed sequence of float32 operations and storage roundings."""
import itertools

import numpy as np
import pytest

from utils import assert_close

SHAPES = [(32, 24, 28, 16), (32, 20, 1), (16, 4), (30, 217, 32)]      # reference tests/test_backend_copy_transpose.py:30-34


def _all_axes(ndim):
    perms = list(itertools.permutations(range(ndim), ndim))
    perms.remove(tuple(range(ndim)))
    return [None] + perms


@pytest.mark.parametrize("shape", SHAPES, ids=[str(s) for s in SHAPES])
def test_copy_transpose_oracle(cpu, shape):
    x = np.random.RandomState(0).uniform(-1, 1, shape).astype(np.float32)
    for ax in _all_axes(len(shape)):
        want = np.transpose(x, axes=ax)
        out = cpu.zeros(want.shape)
        cpu.copy_transpose(cpu.array(x), out, axes=ax)
        assert np.array_equal(out.get(), want)


def test_compensated_sum_oracle_keeps_what_plain_accumulation_loses(cpu):
    """the defining property: 4096 additions of 1e-3 into a float16 accumulator
    starting at 1.0 -- plain accumulation stalls (1e-3 is below half a unit in
    the last place of 4.0), the compensated one stays within one unit in the
    last place of the exact result"""
    n, steps = 64, 4096
    add = np.full((n, n), 1e-3, dtype=np.float16)
    exact = 1.0 + steps * float(np.float16(1e-3))
    s, c, a = cpu.array(np.ones((n, n), np.float16), dtype=np.float16), cpu.zeros((n, n), dtype=np.float16), \
        cpu.array(add, dtype=np.float16)
    plain = np.ones((n, n), np.float16)
    for _ in range(steps):
        cpu.compensated_sum(s, c, a)
        plain = (plain.astype(np.float32) + add.astype(np.float32)).astype(np.float16)
    ulp = float(np.spacing(np.float16(exact)))
    assert np.all(np.abs(s.get().astype(np.float64) - exact) <= ulp)
    assert np.all(np.abs(plain.astype(np.float64) - exact) > 100 * ulp)
    assert c.kahan_count == steps


def test_compensated_sum_oracle_scales_and_reset(cpu):
    rs = np.random.RandomState(1)
    s0, c0, a0 = [rs.rand(8, 8).astype(np.float32) for _ in range(3)]
    s, c, a = cpu.array(s0), cpu.array(c0 * 1e-3), cpu.array(a0)
    cpu.compensated_sum(s, c, a, cmp_scale=0.5, add_scale=-2.0)
    y = a0 * np.float32(-2.0) - (c0 * 1e-3).astype(np.float32) * np.float32(0.5)
    assert np.array_equal(s.get(), s0 + y)
    assert np.array_equal(c.get(), ((s0 + y) - s0) - y)
    # with kahan_reset the compensation term is dropped once the count passes it
    c.kahan_reset, c.kahan_count = 1, 2
    before, cbefore = s.get().copy(), c.get().copy()
    cpu.compensated_sum(s, c, a)
    assert np.array_equal(s.get(), before + a0)
    assert c.kahan_count == 1 and not np.array_equal(s.get(), before + (a0 - cbefore))


# ---- GPU ----------------------------------------------------------------------------------

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", SHAPES, ids=[str(s) for s in SHAPES])
def test_copy_transpose_hip(hip, shape, dtype):
    x = np.random.RandomState(0).uniform(-1, 1, shape).astype(dtype)
    X = hip.array(x, dtype=dtype)
    for ax in _all_axes(len(shape)):
        want = np.transpose(x, axes=ax)
        out = hip.zeros(want.shape, dtype=dtype)
        hip.copy_transpose(X, out, axes=ax)
        assert np.array_equal(out.get(), want), ax


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(1, 1), (1, 77), (77, 1), (65, 63), (129, 1025), (3, 5, 7), (2, 3, 4, 5, 6),
                                   (2000, 3000)], ids=str)
def test_copy_transpose_edges_hip(hip, shape):
    x = np.arange(int(np.prod(shape)), dtype=np.int32).reshape(shape)
    X = hip.array(x, dtype=np.int32)
    out = hip.zeros(shape[::-1], dtype=np.int32)
    hip.copy_transpose(X, out)
    assert np.array_equal(out.get(), x.T)
    if len(shape) == 2:
        # strided source and destination windows
        r, c = shape[0] // 2 + 1, shape[1] // 2 + 1
        big = hip.zeros((c + 3, r + 2), dtype=np.int32)
        hip.copy_transpose(X[:r, :c], big[1:c + 1, 2:r + 2])
        got = big.get()
        assert np.array_equal(got[1:c + 1, 2:r + 2], x[:r, :c].T)
        assert got[0].sum() == 0 and got[:, :2].sum() == 0 and got[c + 1:].sum() == 0


@pytest.mark.gpu
def test_copy_transpose_checks_hip(hip):
    a = hip.zeros((4, 6))
    with pytest.raises(AssertionError):
        hip.copy_transpose(a, hip.zeros((4, 6)))                 # wrong output shape
    with pytest.raises(AssertionError):
        hip.copy_transpose(a, hip.zeros((6, 4), dtype=np.float16))
    with pytest.raises(AssertionError):
        hip.copy_transpose(a, a.T)                               # same memory


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float16, np.float32], ids=["f16", "f32"])
def test_compensated_sum_hip_matches_oracle_bit_for_bit(pair, dtype):
    cpu, hip = pair
    rs = np.random.RandomState(3)
    shape = (200, 333)
    s0 = rs.rand(*shape).astype(dtype)
    adds = [(rs.rand(*shape) * 1e-2).astype(dtype) for _ in range(6)]
    res = []
    for be in pair:
        s, c = be.array(s0, dtype=dtype), be.zeros(shape, dtype=dtype)
        c.kahan_reset = 3
        for k, a in enumerate(adds):
            be.compensated_sum(s, c, be.array(a, dtype=dtype), cmp_scale=1.0, add_scale=1.0 - 0.25 * (k % 2))
        res.append((s.get(), c.get(), c.kahan_count))
    assert np.array_equal(res[1][0], res[0][0])
    assert np.array_equal(res[1][1], res[0][1])
    assert res[1][2] == res[0][2]


@pytest.mark.gpu
def test_compensated_sum_hip_long_run_and_stochastic(hip):
    n, steps = 64, 2048
    s = hip.array(np.ones((n, n), np.float16), dtype=np.float16)
    c = hip.zeros((n, n), dtype=np.float16)
    a = hip.array(np.full((n, n), 1e-3, np.float16), dtype=np.float16)
    for _ in range(steps):
        hip.compensated_sum(s, c, a)
    exact = 1.0 + steps * float(np.float16(1e-3))
    assert np.all(np.abs(s.get().astype(np.float64) - exact) <= float(np.spacing(np.float16(exact))))
    # stochastically rounded accumulator: values stay on the coarse grid, the
    # compensation keeps the mean on target
    s2 = hip.array(np.ones((n, n), np.float16), dtype=np.float16)
    s2.rounding = 6
    c2 = hip.zeros((n, n), dtype=np.float16)
    for _ in range(256):
        hip.compensated_sum(s2, c2, a)
    got = s2.get().astype(np.float32)
    assert np.all((got.view(np.uint32) & np.uint32((1 << 17) - 1)) == 0)
    want = 1.0 + 256 * float(np.float16(1e-3))
    assert abs(got.astype(np.float64).mean() - want) < 2e-3
    assert_close(got, np.full((n, n), want, np.float32), rtol=0, atol=2.0 ** -6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["f32", "f16"])
@pytest.mark.parametrize("shape", [(2048, 1500), (1111, 2003)])
def test_large_transposed_views_are_staged_through_the_tiled_transpose(hip, shape, dtype):
    """x.T of a large tensor as an operand: copied dense first (or straight
    into the output); same values as numpy, also on the replayed second run and
    when the output aliases the operand"""
    be = hip
    rs = np.random.RandomState(shape[0])
    m, n = shape
    a = rs.standard_normal((m, n)).astype(dtype)
    b = rs.standard_normal((n, m)).astype(dtype)
    c = rs.standard_normal((m, n)).astype(dtype)
    ta, tb, tc = be.array(a, dtype=dtype), be.array(b, dtype=dtype), be.array(c, dtype=dtype)
    out = be.empty((n, m), dtype=dtype)
    out32 = be.empty((n, m))
    a32, b32, c32 = (v.astype(np.float32) for v in (a, b, c))
    before = be.plan_stats["launches"]
    for rep in range(2):
        out[:] = ta.T
        assert np.array_equal(out.get(), a.T)
    assert be.plan_stats["launches"] - before == 2          # one tiled copy each, nothing else
    for rep in range(2):
        out32[:] = ta.T + tb
        assert_close(out32.get(), a32.T + b32, rtol=1e-6, atol=1e-6)
        out32[:] = ta.T * tc.T - tb
        assert_close(out32.get(), a32.T * c32.T - b32, rtol=1e-6, atol=1e-6)
        out32[:] = (ta + tc).T
        assert_close(out32.get(), (a32 + c32).T, rtol=1e-6, atol=1e-6)
        out32[:] = be.sum(ta.T, axis=0) + tb
        assert_close(out32.get(), a32.T.sum(axis=0, keepdims=True) + b32, rtol=1e-5, atol=1e-4)
    if dtype == np.float32:
        sq = rs.standard_normal((1600, 1600)).astype(np.float32)
        t = be.array(sq)
        t[:] = t.T + 1.0                                    # the staging copy makes this well defined
        assert np.array_equal(t.get(), sq.T + 1.0)
