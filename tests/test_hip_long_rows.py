"""Axis-1 trees over rows too long for one workgroup's registers: the row
family keeps what it can of an operand -- leading tiles in LDS, the next in the
registers that are left -- and fetches the rest again in every sweep.  Shapes
are chosen to reach every form (plain operand parking beside a resident one,
split residence of a single operand, rows with a partial last tile, the
cooperative variant with few rows) and compared with the oracle on the same
seeded inputs.

Tolerances: fp32 storage 2e-5, fp16 storage 1e-3, both relative to
max(|want|, 1e-3 max|want|); sums over 10^5 terms get the usual allowance for
numpy adding them one after the other."""
import numpy as np
import pytest

from neon_amd import configs
from utils import rel_err

pytestmark = pytest.mark.gpu


def plan_of(hip, issue):
    """the single kernel's generation parameters"""
    with hip.capture() as groups:
        issue()
    assert len(groups) == 1
    return hip.time_group(groups[0], reps=1)[1].spec


def bn_pair(be, x, d, shape, dtype):
    vec = lambda: be.zeros((shape[0], 1))     # noqa: E731
    rs = np.random.RandomState(3)
    gamma = be.array(rs.uniform(0.5, 1.5, (shape[0], 1)).astype(np.float32))
    beta = be.array((rs.standard_normal((shape[0], 1)) * 0.1).astype(np.float32))
    y, dout = be.empty(shape, dtype=dtype), be.empty(shape, dtype=dtype)
    xsum, xvar, gmean, gvar, gg, gb = vec(), vec(), vec(), vec(), vec(), vec()
    be.compound_fprop_bn(x, xsum, xvar, gmean, gvar, gamma, beta, y, 1e-3, 0.9, True)
    be.compound_bprop_bn(dout, gg, gb, d, x, xsum, xvar, gamma, 1e-3)
    return [t.get().astype(np.float64) for t in (y, xsum, xvar, gmean, gvar, dout, gg, gb)]


@pytest.mark.parametrize("shape,dtype", [
    ((200, 100352), np.float16),      # x resident, deltas parked (9 tiles) and held (3)
    ((300, 100352), np.float16),      # the same with more rows than compute units
    ((130, 150528), np.float16),      # 19 tiles: one operand split between LDS and registers
    ((129, 200704), np.float16),      # 25 tiles: registers and LDS exactly full
    ((130, 100003), np.float32),      # fp32, 25 tiles, partial last tile
    ((72, 200704), np.float16),       # few rows: three workgroups per row, each with its share resident
    ((140, 140001), np.float16),      # 18 tiles, partial last tile
    ((64, 401408), np.float16),       # few rows: four workgroups per row cooperate, each parking its share
    ((120, 300000), np.float16),      # two workgroups per row, 19 tiles each: parked, held and fetched again
    ((150, 270000), np.float16),      # 33 tiles: 25 of them kept, the rest streamed by a loop proper in every sweep
    ((140, 600000), np.float16),      # 74 tiles: the same, mostly loop
    ((100, 540001), np.float32),      # two workgroups per row, 66 tiles each, partial last tile
])
def test_batch_norm_pair_over_long_rows(pair, shape, dtype):
    cpu, hip = pair
    rs = np.random.RandomState(shape[1] % 97)
    x0 = (rs.standard_normal(shape) * 2 + 0.5).astype(np.float32).astype(dtype)
    d0 = rs.standard_normal(shape).astype(np.float32).astype(dtype)
    res = []
    for be in pair:
        sdt = np.float32 if be is cpu else dtype            # the oracle computes in fp32 on the quantised values
        res.append(bn_pair(be, be.array(x0.astype(sdt), dtype=sdt), be.array(d0.astype(sdt), dtype=sdt), shape, dtype))
    tol = 1e-3 if dtype == np.float16 else 2e-5
    for got, want, name in zip(res[1], res[0], ("y", "xmean", "xvar", "gmean", "gvar", "delta", "grad_gamma", "grad_beta")):
        if name.startswith("grad"):
            # sums of 10^5 products: numpy adds them in sequence in fp32
            assert np.abs(got - want).max() <= 2e-4 * np.abs(want).max() + 1e-2, name
        else:
            assert rel_err(got, want, floor_frac=1e-3) <= tol, name


def test_which_forms_the_planner_picks(hip):
    """the shapes above really reach the forms they are meant to"""
    f16 = np.float16

    def bprop_spec(shape, dtype):
        x, d, o = hip.empty(shape, dtype=dtype), hip.empty(shape, dtype=dtype), hip.empty(shape, dtype=dtype)
        v = [hip.zeros((shape[0], 1)) for _ in range(5)]
        return plan_of(hip, lambda: hip.compound_bprop_bn(o, v[0], v[1], d, x, v[2], v[3], v[4], 1e-3))

    def fprop_spec(shape, dtype):
        x, o = hip.empty(shape, dtype=dtype), hip.empty(shape, dtype=dtype)
        v = [hip.zeros((shape[0], 1)) for _ in range(6)]
        return plan_of(hip, lambda: hip.compound_fprop_bn(x, v[0], v[1], v[2], v[3], v[4], v[5], o, 1e-3, 0.9, True))

    p = bprop_spec((200, 100352), f16).params
    assert (p["NCH"], p["passing"], p["parked"], p["held"]) == (13, 1, 9, 3)
    p = fprop_spec((130, 150528), f16).params
    assert (p["NCH"], p["passing"], p["parked"], p["held"]) == (19, 1, 9, 10)
    p = fprop_spec((129, 200704), f16).params
    assert (p["NCH"], p["passing"], p["parked"], p["held"]) == (25, 1, 9, 16)
    p = fprop_spec((130, 100003), np.float32).params
    assert (p["NCH"], p["parked"], p["held"], p["tail"]) == (25, 9, 16, True)
    spec = bprop_spec((64, 401408), f16)
    assert spec.family == "rowcoop" and spec.params["parked"] > 0
    spec = bprop_spec((120, 300000), f16)
    assert spec.family == "rowcoop" and spec.params["NCH"] == 19 and spec.params["chunks"] == 2
    assert spec.params["parked"] == 9 and spec.params["passing"] == 2
    spec = fprop_spec((150, 270000), f16)
    assert (spec.params["NCH"], spec.params["parked"], spec.params["held"]) == (33, 9, 16)
    assert "#pragma unroll 1\n    for (int kb = 28; kb < 33; kb += 4)" in spec.source
    spec = bprop_spec((140, 600000), f16)
    assert spec.family == "row" and spec.params["NCH"] == 74 and spec.params["passing"] == 2
    spec = bprop_spec((100, 540001), np.float32)
    assert spec.family == "rowcoop" and (spec.params["NCH"], spec.params["chunks"], spec.params["tail"]) == (66, 2, True)
    # more rows than compute units: the same form (one workgroup per compute unit at a time)
    p = bprop_spec((300, 100352), f16).params
    assert (p["parked"], p["held"], p["passing"]) == (9, 3, 1)


@pytest.mark.parametrize("shape,dtype", [((130, 150528), np.float16), ((130, 100003), np.float32),
                                         ((135, 300001), np.float32), ((20, 1500000), np.float32)])
def test_row_softmax_and_normalisation_over_long_rows(pair, shape, dtype):
    cpu, hip = pair
    rs = np.random.RandomState(5)
    x0 = (rs.standard_normal(shape) * 2).astype(np.float32).astype(dtype)
    gam0 = rs.uniform(0.5, 1.5, (shape[0], 1)).astype(np.float32)
    bet0 = (rs.standard_normal((shape[0], 1)) * 0.1).astype(np.float32)
    res = []
    for be in pair:
        sdt = np.float32 if be is cpu else dtype
        x = be.array(x0.astype(sdt), dtype=sdt)
        sm, nm = be.empty(shape), be.empty(shape, dtype=dtype)
        sm[:] = be.exp(x - be.max(x, axis=1)) / be.sum(be.exp(x - be.max(x, axis=1)), axis=1)
        configs.c4_rownorm(be, nm, x, be.array(gam0), be.array(bet0))
        res.append((sm.get().astype(np.float64), nm.get().astype(np.float64)))
    assert rel_err(res[1][0], res[0][0], floor_frac=1e-3) <= 1e-4           # (numpy's sequential fp32 sum of 10^5 terms)
    x64 = x0.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    assert rel_err(res[1][0], e / e.sum(axis=1, keepdims=True), floor_frac=1e-3) <= 1e-5
    assert rel_err(res[1][1], res[0][1], floor_frac=1e-3) <= (1e-3 if dtype == np.float16 else 2e-5)


@pytest.mark.parametrize("shape", [(8, 300001), (40, 70000)])
def test_variance_of_shared_rows_with_a_large_mean(hip, shape):
    """rows spread over several workgroups, values far from zero (mean 100,
    deviation 1): the parts' second moments are taken around their own means
    and combined exactly, so the variance keeps the accuracy of a two-pass
    evaluation -- against float64"""
    rs = np.random.RandomState(shape[0])
    x = (100.0 + rs.standard_normal(shape)).astype(np.float32)
    x[0, : shape[1] // 2] += 3.0             # parts of one row with different means
    tx = hip.array(x)
    mean, var, out = hip.empty((shape[0], 1)), hip.empty((shape[0], 1)), hip.empty(shape)
    with hip.fused():
        mean[:] = hip.mean(tx, axis=1)
        var[:] = hip.var(tx, axis=1)
        out[:] = (tx - hip.mean(tx, axis=1)) / hip.sqrt(hip.var(tx, axis=1) + 1e-5)
    x64 = x.astype(np.float64)
    m64, v64 = x64.mean(axis=1, keepdims=True), x64.var(axis=1, keepdims=True)
    assert np.abs(mean.get() - m64).max() <= 2e-5
    assert np.abs(var.get() - v64).max() <= 2e-4 * v64.max()
    assert np.abs(out.get() - (x64 - m64) / np.sqrt(v64 + 1e-5)).max() <= 2e-4
    fams = set(p.spec.family for p in hip.plans.values())
    assert "rowcoop" in fams


@pytest.mark.parametrize("shape,dtype", [((6, 300000), np.float32), ((300, 140000), np.float32), ((5, 1200000), np.float16)])
def test_softmax_over_streamed_rows_with_infinities_and_nans(hip, shape, dtype):
    """rows too long for registers take maximum and sum of exponentials in one
    sweep (a running pair): -inf entries, a row of nothing but -inf, a NaN, a
    row whose maximum comes last -- as the three-sweep numpy evaluation has it"""
    rs = np.random.RandomState(41)
    x = (rs.standard_normal(shape) * 3).astype(dtype)
    x[0, 5] = -np.inf
    x[1, :] = -np.inf                        # -inf - -inf: NaN everywhere in the row
    x[2, 77] = np.nan
    x[3, -1] = 60.0                          # the running maximum jumps at the very end
    x[4, 0] = 60.0                           # ... or is there from the start
    tx = hip.array(x, dtype=dtype)
    out, lse = hip.empty(shape), hip.empty((shape[0], 1))
    out[:] = hip.exp(tx - hip.max(tx, axis=1)) / hip.sum(hip.exp(tx - hip.max(tx, axis=1)), axis=1)
    lse[:] = hip.log(hip.sum(hip.exp(tx - hip.max(tx, axis=1)), axis=1)) + hip.max(tx, axis=1)
    x64 = x.astype(np.float64)
    with np.errstate(invalid="ignore"):
        m = x64.max(axis=1, keepdims=True)
        e = np.exp(x64 - m)
        want = e / e.sum(axis=1, keepdims=True)
        want_lse = np.log(e.sum(axis=1, keepdims=True)) + m
    got, got_lse = out.get().astype(np.float64), lse.get().astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    ok = ~np.isnan(want)
    assert np.abs(got[ok] - want[ok]).max() <= 1e-5 * want[ok].max()
    assert got[0, 5] == 0.0
    assert np.array_equal(np.isnan(got_lse), np.isnan(want_lse))
    okl = ~np.isnan(want_lse)
    assert np.abs(got_lse[okl] - want_lse[okl]).max() <= 1e-5 * np.abs(want_lse[okl]).max()


@pytest.mark.parametrize("shape,dtype", [((8, 300001), np.float32), ((20, 1200000), np.float16), ((300, 150000), np.float32)])
def test_softmax_and_normalisation_of_one_operand_in_one_group(hip, shape, dtype):
    """both trees over the same long rows in one fusion group: the running
    (max, sum) pair, the sums and the parts' second moments travel in the same
    sweep and -- where rows are shared -- the same exchange"""
    rs = np.random.RandomState(shape[0])
    x = (rs.standard_normal(shape) * 2 + 1).astype(dtype)
    tx = hip.array(x, dtype=dtype)
    sm, nm = hip.empty(shape), hip.empty(shape)
    before = hip.plan_stats["launches"]
    node = hip._api.OpTreeNode
    # (handed over as one statement group, the way the compound batch-norm calls hand over theirs)
    hip._flush()
    hip._run([node({"op": "assign"}, sm, hip.exp(tx - hip.max(tx, axis=1)) / hip.sum(hip.exp(tx - hip.max(tx, axis=1)), axis=1)),
              node({"op": "assign"}, nm, (tx - hip.mean(tx, axis=1)) / hip.sqrt(hip.var(tx, axis=1) + 1e-5))])
    assert hip.plan_stats["launches"] - before == 1
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=1, keepdims=True))
    want_sm = e / e.sum(axis=1, keepdims=True)
    want_nm = (x64 - x64.mean(axis=1, keepdims=True)) / np.sqrt(x64.var(axis=1, keepdims=True) + 1e-5)
    assert rel_err(sm.get().astype(np.float64), want_sm, floor_frac=1e-3) <= 2e-5
    assert np.abs(nm.get().astype(np.float64) - want_nm).max() <= 2e-4
