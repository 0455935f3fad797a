"""bfloat16 storage with fp32 arithmetic on the hip backend.  The oracle side is
the fp32 CPU oracle on inputs that hold bf16 values exactly, its results rounded
to bf16 by oracle/bf16.py (pinned bit for bit in tests/test_oracle.py).

Tolerance: a bf16 value carries 8 significant bits, so two correct evaluations
that differ in the last fp32 bits may land one bf16 step (2^-8 relative, 3.9e-3)
apart; results are compared to 1e-2 of max(|want|, 1e-3 max|want|) -- the
form used for fp16 storage with its bound scaled to the format."""
import numpy as np
import pytest

from neon_amd import configs
from neon_amd.backends import bfloat16
from neon_amd.backends.hip import bf16 as hostbf16
from oracle.bf16 import round_to_bf16
from utils import rel_err

pytestmark = pytest.mark.gpu
TOL = 1e-2


def _q(a):
    return round_to_bf16(np.asarray(a, dtype=np.float32))


def test_set_get_fill_and_copy_round_trip(hip):
    rs = np.random.RandomState(0)
    x = (rs.standard_normal((33, 70)) * 5).astype(np.float32)
    t = hip.array(x, dtype=bfloat16)
    assert t.dtype == bfloat16 and t.nbytes == 2 * x.size
    got = t.get()
    assert got.dtype == np.float32 and np.array_equal(got.view(np.uint32), _q(x).view(np.uint32))   # host rounding = oracle's
    f = hip.empty((5, 9), dtype=bfloat16)
    f[:] = 1.0 / 3.0
    assert np.array_equal(f.get(), np.full((5, 9), _q([1.0 / 3.0])[0], np.float32))
    # device-side store rounding (fp32 -> bf16 in a kernel) is the same nearest-even
    src = hip.array(x)
    dst = hip.empty(x.shape, dtype=bfloat16)
    dst[:] = src * 1.0
    assert np.array_equal(dst.get().view(np.uint32), _q(x).view(np.uint32))
    back = hip.empty(x.shape)
    back[:] = dst                                                            # widening copy is exact
    assert np.array_equal(back.get(), _q(x))
    assert np.array_equal(dst[3:9, 5:40].get(), _q(x)[3:9, 5:40])            # views


def test_elementwise_and_broadcast_trees(pair):
    cpu, hip = pair
    rs = np.random.RandomState(1)
    shape = (300, 264)
    x, y = _q(rs.standard_normal(shape)), _q(rs.standard_normal(shape) * 2)
    col, row = _q(rs.uniform(0.5, 1.5, (shape[0], 1))), rs.standard_normal((1, shape[1])).astype(np.float32)

    def f(be, X, Y, Cc, Rr):
        return be.tanh(0.5 * X + 2.0 * Y) * Cc - be.maximum(X, Y) / (be.absolute(Rr) + 1.0)

    out = hip.empty(shape, dtype=bfloat16)
    out[:] = f(hip, hip.array(x, dtype=bfloat16), hip.array(y, dtype=bfloat16), hip.array(col, dtype=bfloat16),
               hip.array(row))
    want = cpu.empty(shape)
    want[:] = f(cpu, cpu.array(x), cpu.array(y), cpu.array(col), cpu.array(row))
    assert rel_err(out.get(), _q(want.get()), floor_frac=1e-3) <= TOL
    # a mixed tree: bf16 and fp16 operands, fp32 result (only the inputs were rounded)
    o32 = hip.empty(shape)
    o32[:] = hip.array(x, dtype=bfloat16) * hip.array(y.astype(np.float16), dtype=np.float16) + 1.0
    assert rel_err(o32.get(), x * y.astype(np.float16).astype(np.float32) + 1.0) <= 1e-5


@pytest.mark.parametrize("shape", [(257, 1040), (6000, 96), (40000, 24)])
def test_reductions_along_both_axes(pair, shape):
    cpu, hip = pair
    rs = np.random.RandomState(shape[0])
    x = _q(rs.standard_normal(shape) * 3)
    X, CX = hip.array(x, dtype=bfloat16), cpu.array(x)
    for axis in (0, 1):
        line = (1, shape[1]) if axis == 0 else (shape[0], 1)
        for name in ("sum", "max", "min"):
            got, want = hip.empty(line, dtype=bfloat16), cpu.empty(line)
            got[:] = getattr(hip, name)(X, axis=axis)
            want[:] = getattr(cpu, name)(CX, axis=axis)
            if name == "sum":
                # fp32 accumulation on both sides; the orders differ, then one bf16 rounding
                assert rel_err(got.get(), _q(want.get()), floor_frac=1e-2) <= TOL, (name, axis)
            else:
                assert np.array_equal(got.get(), want.get()), (name, axis)        # exact: values are bf16 already
        am, cam = hip.empty(line, dtype=np.int32), cpu.empty(line, dtype=np.int32)
        am[:] = hip.argmax(X, axis=axis)
        cam[:] = cpu.argmax(CX, axis=axis)
        assert np.array_equal(am.get(), cam.get())
        full, cfull = hip.empty(shape, dtype=bfloat16), cpu.empty(shape)
        full[:] = (X - hip.mean(X, axis=axis)) / hip.sqrt(hip.var(X, axis=axis) + 1e-5)
        cfull[:] = (CX - cpu.mean(CX, axis=axis)) / cpu.sqrt(cpu.var(CX, axis=axis) + 1e-5)
        assert rel_err(full.get(), _q(cfull.get()), floor_frac=1e-3) <= TOL, axis


def test_row_normalisation_config_in_bf16(pair):
    """the fp16 benchmark tree (C4) on bf16 storage, at a shape the oracle takes seconds for"""
    cpu, hip = pair
    shape = (64, 100352)
    rs = np.random.RandomState(4)
    x = _q(rs.standard_normal(shape) * 2.0 + 0.5)
    gamma = rs.uniform(0.5, 1.5, (shape[0], 1)).astype(np.float32)
    beta = (rs.standard_normal((shape[0], 1)) * 0.1).astype(np.float32)
    o = hip.empty(shape, dtype=bfloat16)
    configs.c4_rownorm(hip, o, hip.array(x, dtype=bfloat16), hip.array(gamma), hip.array(beta))
    w = cpu.empty(shape)
    configs.c4_rownorm(cpu, w, cpu.array(x), cpu.array(gamma), cpu.array(beta))
    got = o.get()
    assert rel_err(got, _q(w.get()), floor_frac=1e-3) <= TOL
    # size-independent property: rows have mean beta and standard deviation gamma (to bf16 resolution)
    assert np.allclose(got.mean(axis=1, keepdims=True), beta, atol=5e-3)
    assert np.allclose(got.std(axis=1, keepdims=True), gamma, rtol=1e-2)


def test_batch_norm_pair_over_long_bf16_rows(pair):
    """rows of 19 bf16 tiles: part of an operand parked in LDS, part held in
    registers, the rest fetched again (the forms tests/test_hip_long_rows.py
    covers for fp16 and fp32)"""
    cpu, hip = pair
    shape = (130, 150528)
    rs = np.random.RandomState(8)
    x = _q(rs.standard_normal(shape) * 2.0 + 0.5)
    d = _q(rs.standard_normal(shape))
    gam = rs.uniform(0.5, 1.5, (shape[0], 1)).astype(np.float32)
    bet = (rs.standard_normal((shape[0], 1)) * 0.1).astype(np.float32)
    res = []
    for be, dt in ((cpu, np.float32), (hip, bfloat16)):
        vec = lambda: be.zeros((shape[0], 1))     # noqa: E731
        X, D = be.array(x, dtype=dt), be.array(d, dtype=dt)
        y, dout = be.empty(shape, dtype=dt), be.empty(shape, dtype=dt)
        xsum, xvar, gmean, gvar, gg, gb = vec(), vec(), vec(), vec(), vec(), vec()
        be.compound_fprop_bn(X, xsum, xvar, gmean, gvar, be.array(gam), be.array(bet), y, 1e-3, 0.9, True)
        be.compound_bprop_bn(dout, gg, gb, D, X, xsum, xvar, be.array(gam), 1e-3)
        res.append([t.get().astype(np.float64) for t in (y, dout, xsum, xvar, gg, gb)])
    for k, name in enumerate(("y", "delta")):
        assert rel_err(res[1][k], _q(res[0][k]), floor_frac=1e-3) <= TOL, name
    for k, name in ((2, "mean"), (3, "var")):
        assert rel_err(res[1][k], res[0][k], floor_frac=1e-3) <= 2e-5, name
    for k, name in ((4, "grad_gamma"), (5, "grad_beta")):
        assert np.abs(res[1][k] - res[0][k]).max() <= 2e-4 * np.abs(res[0][k]).max() + 1e-2, name


def test_stochastic_rounding_into_bf16_is_unbiased(hip):
    x = np.full((64, 4096), 1.0 + 2.0 ** -10, np.float32)            # a quarter of the way between two 4-bit neighbours
    t = hip.empty(x.shape, dtype=bfloat16)
    t.rounding = 4
    t[:] = hip.array(x) * 1.0
    got = t.get()
    lo, hi = 1.0, 1.0 + 2.0 ** -4
    assert set(np.unique(got)) <= {np.float32(lo), np.float32(hi)}
    p_hi = (got == hi).mean()
    assert abs(p_hi - (2.0 ** -10) / (2.0 ** -4)) < 5e-3
    assert hostbf16.is_bfloat16(t.dtype)
