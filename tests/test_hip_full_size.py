"""The benchmark configurations at their FULL shapes against the CPU oracle
(same seeded inputs, same op-trees: neon_amd/configs.py), plus the rewritten and
the as-written forms of the softmax / cross-entropy trees side by side.

Tolerances: integer results bit-exact; fp32 1e-5 relative; fp16 storage 1e-3 of
max(|want|, 1e-3 max|want|) (values near a row's mean are tiny, one fp16 step of
the store would dominate otherwise).  The sum of 32000 exponentials is added
in another order than numpy's (and, in the one-sweep form, rescaled by
exp(m - M) factors): it is compared to 1e-5 as well, and against float64."""
import contextlib

import numpy as np
import pytest

from neon_amd import configs
from neon_amd.backends.backend import Block
from neon_amd.backends.hip import optree_ir
from utils import assert_close, rel_err

pytestmark = pytest.mark.gpu


@contextlib.contextmanager
def rewrites(hip, online_lse, onehot_gather):
    """run a block with the tree rewrites switched as given (they are part of a
    program's key, so both forms get their own kernels)"""
    old = optree_ir.ONLINE_LSE, optree_ir.ONEHOT_GATHER
    optree_ir.ONLINE_LSE, optree_ir.ONEHOT_GATHER = online_lse, onehot_gather
    hip.synchronize()
    hip._launch_cache.clear()
    try:
        yield
    finally:
        optree_ir.ONLINE_LSE, optree_ir.ONEHOT_GATHER = old
        hip.synchronize()
        hip._launch_cache.clear()


def test_c1_and_c2_full_size(pair):
    cpu, hip = pair
    x, y = configs.inputs_c1()
    res = []
    for be in pair:
        X, Y, out, fused = be.array(x), be.array(y), be.empty(x.shape), be.empty(x.shape)
        configs.c1a(be, out, X, Y)
        configs.c1b(be, out)
        configs.c1_fused(be, fused, X, Y)
        res.append((out.get(), fused.get()))
    for g, w in zip(res[1], res[0]):
        assert_close(g, w, rtol=1e-5, atol=1e-7)
    (x2,) = configs.inputs_c2()
    want = cpu.empty(x2.shape)
    configs.c2_softmax(cpu, want, cpu.array(x2))
    for lse in (True, False):
        with rewrites(hip, lse, True):
            got = hip.empty(x2.shape)
            configs.c2_softmax(hip, got, hip.array(x2))
            assert_close(got.get(), want.get(), rtol=1e-5, atol=1e-9, what="softmax, one-sweep pair %s" % lse)
            assert np.allclose(got.get().sum(axis=0), 1.0, atol=2e-6)


def test_c3_ten_fused_adam_steps_full_size(pair):
    cpu, hip = pair
    grad, param = configs.inputs_c3()
    res = []
    for be in pair:
        bsz, be.bsz = be.bsz, 1
        g, p = be.array(grad), be.array(param)
        m, v = be.zeros(configs.C3_SHAPE), be.zeros(configs.C3_SHAPE)
        first = None
        for t in range(1, 11):
            be.begin(Block.update, t)
            configs.c3_adam_step(be, p, g, m, v, t)
            be.end(Block.update, t)
            if t == 1:
                first = (p.get(), m.get(), v.get())
        res.append((first, (p.get(), m.get(), v.get())))
        be.bsz = bsz
        del g, p, m, v
    for step in (0, 1):
        for k, name in enumerate(("param", "m", "v")):
            assert_close(res[1][step][k], res[0][step][k], rtol=1e-5, atol=1e-12,
                         what="%s after step %d" % (name, (1, 10)[step]))


def test_c4_row_normalisation_full_size(pair):
    cpu, hip = pair
    x, gamma, beta = configs.inputs_c4()
    o_cpu = cpu.empty(configs.C4_SHAPE, dtype=np.float16)
    # oracle: the fp16 values held in fp32 (numpy would evaluate fp16 operands in fp16), fp32 arithmetic, fp16 store
    configs.c4_rownorm(cpu, o_cpu, cpu.array(x.astype(np.float32)), cpu.array(gamma), cpu.array(beta))
    o_hip = hip.empty(configs.C4_SHAPE, dtype=np.float16)
    configs.c4_rownorm(hip, o_hip, hip.array(x, dtype=np.float16), hip.array(gamma), hip.array(beta))
    want, got = o_cpu.get().astype(np.float64), o_hip.get().astype(np.float64)
    assert rel_err(got, want, floor_frac=1e-3) <= 1e-3
    # ... and the fraction of results that differ from the oracle's at all stays small
    # (two correct fp32 evaluations can round to neighbouring fp16 values)
    assert (got != want).mean() < 0.02


def test_c5_full_size_all_forms(pair):
    cpu, hip = pair
    x, idx = configs.inputs_c5()
    cx, ci = cpu.array(x), cpu.array(idx, dtype=np.int32)
    cam, cmx, cce = cpu.empty((1, 256), dtype=np.int32), cpu.empty((1, 256)), cpu.empty((1, 256))
    configs.c5a_argmax(cpu, cam, cx)
    configs.c5b_max(cpu, cmx, cx)
    t = cpu.empty(x.shape)
    t[:] = cpu.onehot(ci, axis=0)
    configs.c5c_cross_entropy(cpu, cce, cx, t)
    x64 = x.astype(np.float64)
    m64 = x64.max(axis=0)
    ce64 = np.log(np.exp(x64 - m64).sum(axis=0)) + m64 - x64[idx.ravel(), np.arange(256)]
    assert_close(cce.get().ravel(), ce64, rtol=1e-5, atol=1e-5, what="oracle against float64")

    hx, hi = hip.array(x), hip.array(idx, dtype=np.int32)
    am, mx = hip.empty((1, 256), dtype=np.int32), hip.empty((1, 256))
    configs.c5a_argmax(hip, am, hx)
    configs.c5b_max(hip, mx, hx)
    assert np.array_equal(am.get(), cam.get()) and np.array_equal(mx.get(), cmx.get())
    with hip.fused():                                    # both from one pass over the logits
        configs.c5a_argmax(hip, am, hx)
        configs.c5b_max(hip, mx, hx)
    assert np.array_equal(am.get(), cam.get()) and np.array_equal(mx.get(), cmx.get())

    families = {}
    for lse, gather in ((True, True), (True, False), (False, True), (False, False)):
        with rewrites(hip, lse, gather):
            ce = hip.empty((1, 256))
            configs.c5c_cross_entropy(hip, ce, hx, hip.onehot(hi, axis=0))
            got = ce.get()
            with hip.capture() as groups:                   # which kernel family ran it
                configs.c5c_cross_entropy(hip, ce, hx, hip.onehot(hi, axis=0))
            families[(lse, gather)] = [hip.time_group(trees, reps=1)[1].spec.family for trees in groups]
            assert_close(got, cce.get(), rtol=1e-5, atol=1e-6, what="cross-entropy, pair %s gather %s" % (lse, gather))
            assert_close(got.ravel(), ce64, rtol=1e-5, atol=1e-5, what="cross-entropy against float64")
            # the dense one-hot form (what neon's cost layer is handed): same tree, t from memory
            dense = hip.empty(x.shape)
            dense[:] = hip.onehot(hi, axis=0)
            configs.c5c_cross_entropy(hip, ce, hx, dense)
            assert_close(ce.get(), cce.get(), rtol=1e-5, atol=1e-6, what="dense one-hot, pair %s" % lse)
    assert families[(True, True)] == ["colsplit"]        # one pass, nobody waits
    assert families[(False, False)] == ["colcoop"]       # three sweeps over resident rows, as written


def test_axis0_trees_too_large_for_one_kernel_are_staged_with_their_reductions_together(pair):
    """A matrix too tall for one workgroup's registers and too large for the
    cooperative family: the reductions of the tree (nested or side by side)
    run as ONE kernel over the operand, then the elementwise rest -- softmax
    reads x twice and writes once.  Against the oracle and float64."""
    cpu, hip = pair
    shape = (9000, 3072)
    rs = np.random.RandomState(77)
    x = (rs.standard_normal(shape) * 3.0).astype(np.float32)
    x64 = x.astype(np.float64)
    e64 = np.exp(x64 - x64.max(axis=0))
    sm64 = e64 / e64.sum(axis=0)
    hx, cx = hip.array(x), cpu.array(x)
    hout, cout = hip.empty(shape), cpu.empty(shape)

    def launches(issue):
        before = hip.plan_stats["launches"]
        issue()
        return hip.plan_stats["launches"] - before

    for name, tree in (("softmax as written", lambda be, t: be.exp(t - be.max(t, axis=0)) /
                        be.sum(be.exp(t - be.max(t, axis=0)), axis=0)),
                       ("softmax, reciprocal form", lambda be, t: be.fprop_softmax(t, 0))):
        cout[:] = tree(cpu, cx)
        for lse, want_launches in ((True, 2), (False, 3)):
            with rewrites(hip, lse, True):
                assert launches(lambda: hout.__setitem__(slice(None), tree(hip, hx))) == want_launches, name
                got = hout.get()
                # numpy adds the 9000 terms of a column one after the other in fp32 (error up to
                # rows x 2^-24); the device adds a tree and stays within 1e-5 of float64
                assert rel_err(got, cout.get(), floor_frac=1e-3) < 1e-4, name
                assert rel_err(got, sm64, floor_frac=1e-3) < 1e-5, name
                assert np.allclose(got.sum(axis=0), 1.0, atol=1e-5)
                # again: the recorded launches (three temporaries' worth of them) are replayed
                hout.fill(0)
                assert launches(lambda: hout.__setitem__(slice(None), tree(hip, hx))) == want_launches
                assert np.array_equal(hout.get(), got)
    # log-softmax: the same two reductions under another elementwise rest
    with rewrites(hip, True, True):
        n = launches(lambda: hout.__setitem__(
            slice(None), hx - hip.max(hx, axis=0) - hip.log(hip.sum(hip.exp(hx - hip.max(hx, axis=0)), axis=0))))
        assert n == 2
        want = x64 - x64.max(axis=0) - np.log(e64.sum(axis=0))
        assert_close(hout.get(), want, rtol=1e-5, atol=2e-5, what="log-softmax")
    # two reductions side by side (no nesting): one pass for both
    n = launches(lambda: hout.__setitem__(slice(None), (hx - hip.min(hx, axis=0)) /
                                          (hip.max(hx, axis=0) - hip.min(hx, axis=0))))
    assert n <= 2
    want = (x64 - x64.min(axis=0)) / (x64.max(axis=0) - x64.min(axis=0))
    assert_close(hout.get(), want, rtol=1e-5, atol=1e-6, what="min-max scaling")
    # nested reductions no family takes together (variance around the mean): one kernel each
    cout[:] = (cx - cpu.mean(cx, axis=0)) / cpu.sqrt(cpu.var(cx, axis=0) + 1e-5)
    n = launches(lambda: hout.__setitem__(slice(None), (hx - hip.mean(hx, axis=0)) /
                                          hip.sqrt(hip.var(hx, axis=0) + 1e-5)))
    assert n == 3
    assert_close(hout.get(), cout.get(), rtol=1e-4, atol=1e-5, what="column normalisation")


def test_all_configurations_against_formulas_written_in_numpy_float64(hip):
    """The five configurations at full shape against the formulas themselves,
    evaluated in numpy float64 with nothing of this package between the inputs
    and the expected values (the oracle shares its op builders with the
    product; this test does not).  fp32 results within 1e-5 (sums of many terms
    with the 2 eps sum|x| allowance), fp16 storage within one fp16 step, indices
    and maxima bit for bit."""
    be = hip
    # C1: 0.5 x + 2 y, then the logistic function in place; and both as one statement
    x, y = configs.inputs_c1()
    X, Y, out, fused = be.array(x), be.array(y), be.empty(x.shape), be.empty(x.shape)
    configs.c1a(be, out, X, Y)
    lin = out.get()
    assert np.array_equal(lin, np.float32(0.5) * x + np.float32(2.0) * y)          # two exact scalings and one rounding
    configs.c1b(be, out)
    configs.c1_fused(be, fused, X, Y)
    sig = 1.0 / (1.0 + np.exp(-(0.5 * x.astype(np.float64) + 2.0 * y.astype(np.float64))))
    assert_close(out.get(), sig, rtol=1e-5, atol=1e-7, what="C1b")
    assert_close(fused.get(), sig, rtol=1e-5, atol=1e-7, what="C1 fused")
    # C2: softmax down the columns
    (x2,) = configs.inputs_c2()
    o2 = be.empty(x2.shape)
    configs.c2_softmax(be, o2, be.array(x2))
    e = np.exp(x2.astype(np.float64) - x2.astype(np.float64).max(axis=0))
    assert_close(o2.get(), e / e.sum(axis=0), rtol=1e-5, atol=1e-9, what="C2")
    # C3: three Adam steps, float64 state carried alongside
    grad, param = configs.inputs_c3()
    p, g, m, v = be.array(param), be.array(grad), be.zeros(param.shape), be.zeros(param.shape)
    p64, g64 = param.astype(np.float64), grad.astype(np.float64)
    m64, v64 = np.zeros_like(p64), np.zeros_like(p64)
    a = configs.ADAM
    for t in range(1, 4):
        be.begin(Block.update, t)
        configs.c3_adam_step(be, p, g, m, v, t)
        be.end(Block.update, t)
        l = a["lr"] * np.sqrt(1 - a["beta2"] ** t) / (1 - a["beta1"] ** t)
        m64 = m64 * a["beta1"] + (1. - a["beta1"]) * g64
        v64 = v64 * a["beta2"] + (1. - a["beta2"]) * g64 * g64
        p64 = p64 - (l * m64) / (np.sqrt(v64) + a["eps"])
    assert_close(m.get(), m64, rtol=1e-5, atol=1e-9, what="C3 m")
    assert_close(v.get(), v64, rtol=1e-5, atol=1e-12, what="C3 v")
    assert_close(p.get(), p64, rtol=1e-5, atol=1e-7, what="C3 param")
    del p, g, m, v, p64, g64, m64, v64
    # C4: row normalisation of fp16 data, fp16 result
    x4, gamma, beta = configs.inputs_c4()
    o4 = be.empty(x4.shape, dtype=np.float16)
    configs.c4_rownorm(be, o4, be.array(x4, dtype=np.float16), be.array(gamma), be.array(beta))
    x64 = x4.astype(np.float64)
    want = gamma * (x64 - x64.mean(axis=1, keepdims=True)) / np.sqrt(x64.var(axis=1, keepdims=True) + 1e-5) + beta
    got = o4.get().astype(np.float64)
    scale = np.maximum(np.abs(want), 1e-3 * np.abs(want).max())
    assert (np.abs(got - want) / scale).max() < 1e-3
    del o4, x64, want, got
    # C5: argmax, max, cross-entropy down 32000 rows
    x5, idx = configs.inputs_c5()
    X5 = be.array(x5)
    am, mx, ce = be.empty((1, 256), dtype=np.int32), be.empty((1, 256)), be.empty((1, 256))
    configs.c5a_argmax(be, am, X5)
    configs.c5b_max(be, mx, X5)
    configs.c5c_cross_entropy(be, ce, X5, be.onehot(be.array(idx, dtype=np.int32), axis=0))
    assert np.array_equal(am.get().ravel(), x5.argmax(axis=0))
    assert np.array_equal(mx.get().ravel(), x5.max(axis=0))
    x64 = x5.astype(np.float64)
    m64 = x64.max(axis=0)
    ce64 = np.log(np.exp(x64 - m64).sum(axis=0)) + m64 - x64[idx.ravel(), np.arange(256)]
    assert_close(ce.get().ravel(), ce64, rtol=1e-5, atol=1e-5, what="C5c")
