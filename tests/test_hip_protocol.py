"""The inter-workgroup hand-off of the split and cooperative kernel families
(``colsplit`` ticket, ``colcoop`` / ``rowcoop`` waiting exchanges): a long
alternating run on fresh data against numpy, and the host's handling of a
cooperative kernel that gave up waiting."""
import numpy as np
import pytest

from neon_amd.backends.hip import planner
from neon_amd.backends.hip import runtime as hiprt
from utils import assert_close


def _families(hip):
    return set(p.spec.family for p in hip.plans.values())


@pytest.mark.gpu
def test_soak_alternating_split_and_cooperative_launches(hip, monkeypatch):
    """2800 launches, three families in turn, new random data every round
    (drawn on the device); max / argmax bit-exact against numpy, sums against
    float64; stops at the first mismatch"""
    # (matrices this small are evaluated in stages otherwise; the protocol is what is under test)
    monkeypatch.setattr(planner, "COLCOOP_MIN_BYTES", 0)
    xs = hip.empty((2048, 128))          # colsplit: one level, one value per column
    xc = hip.empty((20000, 64))          # colcoop: two levels over more rows than a workgroup holds
    xr = hip.empty((8, 40000))           # rowcoop: few very long rows
    am, mx = hip.empty((1, 128), dtype=np.int32), hip.empty((1, 128))
    lse, devc = hip.empty((1, 64)), hip.empty((20000, 64))
    rs_, dev = hip.empty((8, 1)), hip.empty((8, 40000))
    for rnd in range(700):
        for t in (xs, xc, xr):
            t[:] = hip.rand() * 8.0 - 4.0
        am[:] = hip.argmax(xs, axis=0)
        mx[:] = hip.max(xs, axis=0)
        lse[:] = hip.sum(hip.exp(xc - hip.max(xc, axis=0)), axis=0)
        devc[:] = xc - hip.mean(xc, axis=0)       # a result of the operand's shape: every workgroup waits for the column sums
        rs_[:] = hip.sum(xr, axis=1)
        dev[:] = xr - hip.mean(xr, axis=1)
        hs, hc, hr = xs.get(), xc.get().astype(np.float64), xr.get().astype(np.float64)
        assert np.array_equal(am.get(), hs.argmax(axis=0).reshape(1, -1).astype(np.int32)), "argmax, round %d" % rnd
        assert np.array_equal(mx.get(), hs.max(axis=0, keepdims=True)), "max, round %d" % rnd
        want = np.exp(hc - hc.max(axis=0, keepdims=True)).sum(axis=0, keepdims=True)
        assert_close(lse.get(), want, rtol=1e-5, atol=0, what="sum exp, round %d" % rnd)
        assert_close(devc.get(), hc - hc.mean(axis=0, keepdims=True), rtol=1e-5, atol=1e-5,
                     what="column deviation, round %d" % rnd)
        assert_close(rs_.get(), hr.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-3, what="row sum, round %d" % rnd)
        assert_close(dev.get(), hr - hr.mean(axis=1, keepdims=True), rtol=1e-5, atol=1e-5,
                     what="row deviation, round %d" % rnd)
    assert {"colsplit", "colcoop", "rowcoop"} <= _families(hip)


@pytest.mark.gpu
def test_the_hand_offs_built_with_release_and_acquire_fences(hip, monkeypatch):
    """the variant parts other than gfx950 get by default (device-scope release
    before a counter update, acquire after reading it): the same three
    families, compiled with it, against numpy"""
    monkeypatch.setattr(planner, "COLCOOP_MIN_BYTES", 0)
    hip.synchronize()
    kernels, plans, cache = hip.kernels, hip.plans, dict(hip._launch_cache)
    hip.kernels = planner.KernelCache(kernels.arch, formal_fences=True)
    assert hip.kernels.formal_fences and "#define NH_FORMAL_FENCES 1" in hip.kernels.header
    hip.plans = {}
    hip._launch_cache.clear()
    try:
        xs, xc, xr = hip.empty((2048, 128)), hip.empty((20000, 64)), hip.empty((8, 40000))
        am, mx = hip.empty((1, 128), dtype=np.int32), hip.empty((1, 128))
        devc, dev = hip.empty((20000, 64)), hip.empty((8, 40000))
        for rnd in range(3):
            for t in (xs, xc, xr):
                t[:] = hip.rand() * 8.0 - 4.0
            am[:] = hip.argmax(xs, axis=0)
            mx[:] = hip.max(xs, axis=0)
            devc[:] = xc - hip.mean(xc, axis=0)
            dev[:] = xr - hip.mean(xr, axis=1)
            hs, hc, hr = xs.get(), xc.get().astype(np.float64), xr.get().astype(np.float64)
            assert np.array_equal(am.get(), hs.argmax(axis=0).reshape(1, -1).astype(np.int32))
            assert np.array_equal(mx.get(), hs.max(axis=0, keepdims=True))
            assert_close(devc.get(), hc - hc.mean(axis=0, keepdims=True), rtol=1e-5, atol=1e-5)
            assert_close(dev.get(), hr - hr.mean(axis=1, keepdims=True), rtol=1e-5, atol=1e-5)
        assert {"colsplit", "colcoop", "rowcoop"} <= _families(hip)
    finally:
        hip.synchronize()
        for plan in hip.plans.values():
            for p_ in (plan if isinstance(plan, list) else [plan]):
                p_.release()
        hip.kernels, hip.plans = kernels, plans
        hip._launch_cache.clear()
        hip._launch_cache.update(cache)


@pytest.mark.gpu
@pytest.mark.parametrize("family", ["colcoop", "rowcoop", "colsplit"])
def test_a_cooperative_kernel_that_gave_up_is_reported_and_replaced(pair, family, monkeypatch):
    """Nothing is made to hang: the word an aborting workgroup would leave is
    written into the plan's workspace from the host.  The next synchronisation
    raises, and from then on the tree runs without inter-workgroup waits."""
    monkeypatch.setattr(planner, "COLCOOP_MIN_BYTES", 0)      # a small matrix, cooperating all the same
    cpu, hip = pair
    rs = np.random.RandomState(9)
    if family == "colcoop":
        x = (rs.standard_normal((20000, 48)) * 2).astype(np.float32)

        def run(be):
            X, out = be.array(x), be.empty(x.shape)
            out[:] = be.exp(X - be.max(X, axis=0)) / be.sum(be.exp(X - be.max(X, axis=0)), axis=0)
            return out
    elif family == "colsplit":
        # (the split family's tagged form: only the last workgroups of a strip wait)
        x = (rs.standard_normal((32000, 256)) * 2).astype(np.float32)

        def run(be):
            X, out = be.array(x), be.empty((1, x.shape[1]))
            out[:] = be.sum(be.exp(X - be.max(X, axis=0)), axis=0)
            return out
    else:
        x = (rs.standard_normal((6, 50000)) * 2).astype(np.float32)

        def run(be):
            X, out = be.array(x), be.empty(x.shape)
            out[:] = (X - be.mean(X, axis=1)) / be.sqrt(be.var(X, axis=1) + 1e-5)
            return out
    want = run(cpu).get()
    hip.synchronize()
    before = set(hip.plans)
    assert_close(run(hip).get(), want, rtol=1e-5, atol=1e-6, what=family)
    fresh = [hip.plans[k] for k in hip.plans if k not in before and hip.plans[k].spec.family == family]
    assert len(fresh) == 1, "the tree should have run as one %s kernel" % family
    plan = fresh[0]
    hip.rt.memset(plan.status_ptr, 0xDEAD, 1, 4)
    out = run(hip)                                   # runs normally, but the plan carries the mark
    with pytest.raises(hiprt.HipError) as err:
        hip.synchronize()
    assert err.value.code == hiprt.NH_ECOOP
    assert plan.key in hip._coop_failed and plan.key not in hip.plans
    hip.synchronize()                                # reported once
    again = run(hip)
    got = again.get()
    assert_close(got, want, rtol=1e-5, atol=1e-6, what=family + " after the fallback")
    # (a split column reduction among the replacement's stages may finish through tagged records: only the
    # strip's last workgroups wait there, for workgroups that started before them, so it does not need the
    # whole grid resident; the program that gave up itself is planned without any wait)
    fresh = dict((k, p) for k, p in hip.plans.items() if k not in before)
    assert all(p.spec.family not in ("colcoop", "rowcoop") for p in fresh.values()), \
        "the replacement must not need all its workgroups resident at once"
    if plan.key in fresh:
        assert fresh[plan.key].status_ptr is None
    del out


@pytest.mark.gpu
def test_a_replayed_cooperative_statement_is_still_checked(hip):
    """the same statement over the same tensors is served from its recording
    (by the C replayer where it is built): the plan must be looked at by the
    next synchronisation all the same"""
    rs = np.random.RandomState(4)
    x = rs.standard_normal((31000, 256)).astype(np.float32)
    X, out = hip.array(x), hip.empty((1, 256))
    with hip.capture() as groups:
        out[:] = hip.max(X, axis=0)
    plan = hip.time_group(groups[0], reps=1)[1]
    assert plan.spec.family == "colsplit" and plan.spec.params["lookback"] and plan.status_ptr is not None
    for _ in range(3):
        out[:] = hip.max(X, axis=0)
    hip.synchronize()
    assert np.array_equal(out.get(), x.max(axis=0, keepdims=True))
    replayed = hip.plan_stats["replayed"]
    assert not hip._coop_pending
    out[:] = hip.max(X, axis=0)
    assert hip.plan_stats["replayed"] == replayed + 1 and hip._coop_pending.get(plan.key) is plan
    hip.synchronize()
    assert not hip._coop_pending
    hip.rt.memset(plan.status_ptr, 0xDEAD, 1, 4)
    out[:] = hip.max(X, axis=0)
    with pytest.raises(hiprt.HipError) as err:
        hip.synchronize()
    assert err.value.code == hiprt.NH_ECOOP and plan.key not in hip.plans
    out[:] = hip.max(X, axis=0)                      # planned again, in the form that never waits
    assert np.array_equal(out.get(), x.max(axis=0, keepdims=True))
    again = hip.plans[plan.key]
    assert again is not plan and again.status_ptr is None and not again.spec.params["lookback"]
