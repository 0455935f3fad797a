"""Parameter-update statement groups (the bodies of the reference's optimizers,
neon/optimizers/optimizer.py, written from their formulas in tests/clients.py)
between ``be.begin(Block.update)`` / ``be.end(Block.update)``: each rule against
a float64 numpy restatement on the oracle (the idiom of the reference's
tests/test_optimizer.py:280-299), and on the GPU against the oracle, where the
whole group must run as ONE fused kernel."""
import numpy as np
import pytest

import clients
from utils import assert_close

SHAPE = (37, 53)


def _np_adam(p, g, m, v, t, bsz, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8):
    g = g / bsz
    m = m * b1 + (1 - b1) * g
    v = v * b2 + (1 - b2) * g * g
    p = p - (lr * np.sqrt(1 - b2 ** t) / (1 - b1 ** t)) * m / (np.sqrt(v) + eps)
    return p, m, v


def _np_momentum(p, g, vel, bsz, lr=0.1, mom=0.9, wd=0.0005):
    vel = mom * vel - lr * (g / bsz + wd * p)
    return p + vel, vel


def _np_rmsprop(p, g, s, bsz, lr=2e-3, decay=0.95, eps=1e-6):
    g = g / bsz
    s = decay * s + g * g * (1 - decay)
    return p - g * lr / (np.sqrt(s + eps) + eps), s


def _np_adadelta(p, g, gsq, dsq, bsz, decay=0.95, eps=1e-6):
    g = g / bsz
    gsq = gsq * decay + (1 - decay) * g * g
    d = np.sqrt((dsq + eps) / (gsq + eps)) * g
    dsq = dsq * decay + (1 - decay) * d * d
    return p - d, gsq, dsq, d


def _draw(nstates, seed=0, shape=SHAPE):
    rs = np.random.RandomState(seed)
    p = rs.standard_normal(shape).astype(np.float32)
    g = (rs.standard_normal(shape) * 0.1).astype(np.float32)
    states = [np.abs(rs.standard_normal(shape) * 0.01).astype(np.float32) for _ in range(nstates)]
    return p, g, states


def _apply(be, rule, steps=3, seed=0, shape=SHAPE, dtype=np.float32, quantise=None):
    nstates = {"adam": 2, "momentum": 1, "rmsprop": 1, "adadelta": 3}[rule]
    p, g, st = _draw(nstates, seed, shape)
    if quantise is not None:
        p, g, st = p.astype(quantise), g.astype(quantise), [s.astype(quantise) for s in st]
    P, G = be.array(p, dtype=dtype), be.array(g, dtype=dtype)
    S = [be.array(s, dtype=dtype) for s in st]
    for t in range(1, steps + 1):
        if rule == "adam":
            clients.adam_update(be, P, G, S[0], S[1], t)
        elif rule == "momentum":
            clients.momentum_update(be, P, G, S[0])
        elif rule == "rmsprop":
            clients.rmsprop_update(be, P, G, S[0])
        else:
            clients.adadelta_update(be, P, G, S[0], S[1], S[2])
    return [P.get()] + [s.get() for s in S]


def _expected(rule, steps=3, seed=0, bsz=128):
    nstates = {"adam": 2, "momentum": 1, "rmsprop": 1, "adadelta": 3}[rule]
    p, g, st = _draw(nstates, seed)
    p, g = p.astype(np.float64), g.astype(np.float64)
    st = [s.astype(np.float64) for s in st]
    for t in range(1, steps + 1):
        if rule == "adam":
            p, st[0], st[1] = _np_adam(p, g, st[0], st[1], t, bsz)
        elif rule == "momentum":
            p, st[0] = _np_momentum(p, g, st[0], bsz)
        elif rule == "rmsprop":
            p, st[0] = _np_rmsprop(p, g, st[0], bsz)
        else:
            p, st[0], st[1], st[2] = _np_adadelta(p, g, st[0], st[1], bsz)
    return [p] + st


RULES = ["adam", "momentum", "rmsprop", "adadelta"]


@pytest.mark.parametrize("rule", RULES)
def test_rule_matches_float64_numpy_on_the_oracle(cpu, rule):
    for got, want in zip(_apply(cpu, rule), _expected(rule)):
        assert_close(got, want.astype(np.float32), rtol=2e-5, atol=1e-7, what=rule)


@pytest.mark.gpu
@pytest.mark.parametrize("rule", RULES)
def test_rule_hip_matches_oracle_as_one_kernel(pair, rule):
    cpu, hip = pair
    want = _apply(cpu, rule, shape=(300, 257), seed=3)
    before = hip.plan_stats["launches"]
    got = _apply(hip, rule, shape=(300, 257), seed=3)
    assert hip.plan_stats["launches"] - before == 3, "each update group must be a single launch"
    for g, w in zip(got, want):
        assert_close(g, w, rtol=1e-5, atol=1e-7, what=rule)


@pytest.mark.gpu
def test_adam_fp16_parameters_hip_matches_oracle(pair):
    """fp16 storage, fp32 arithmetic: the oracle evaluates the step in fp32 on
    the fp16-quantised inputs (numpy would compute fp16 operands in fp16) and
    its results are rounded to fp16 once, like the device's stores"""
    cpu, hip = pair
    want = _apply(cpu, "adam", steps=1, shape=(64, 520), seed=5, quantise=np.float16)
    got = _apply(hip, "adam", steps=1, shape=(64, 520), seed=5, dtype=np.float16)
    for g, w in zip(got, want):
        assert g.dtype == np.float16
        # the parameter is computed from m and v after THEIR rounding to fp16 on the
        # device (a later statement reads what an earlier one stored): 1e-3 relative
        assert_close(g.astype(np.float32), w.astype(np.float16).astype(np.float32), rtol=1e-3, atol=1e-6,
                     what="adam f16")


@pytest.mark.gpu
def test_statements_inside_a_minibatch_block_fuse_and_keep_program_order(pair):
    """The reference brackets every minibatch with begin / end(Block.minibatch)
    (models/model.py:204-217): inside, consecutive elementwise statements over
    one shape run as one kernel, and whatever is not such a statement -- a
    product, a copy to the host, a reduction -- sees what the program wrote
    before it.  The sequence below (bias + activation, a product, a momentum
    update of two parameters, a host read in the middle) against the oracle
    and against the same sequence outside any block."""
    from neon_amd.backends.backend import Block
    rs = np.random.RandomState(11)
    w0, x0, b0 = rs.standard_normal((64, 48)).astype(np.float32), rs.standard_normal((48, 32)).astype(np.float32), \
        rs.standard_normal((64, 1)).astype(np.float32)
    g0, g1 = rs.standard_normal((64, 48)).astype(np.float32), rs.standard_normal((64, 1)).astype(np.float32)

    def program(be, block):
        w, x, b = be.array(w0), be.array(x0), be.array(b0)
        gw, gb = be.array(g0), be.array(g1)
        vw, vb = be.zeros((64, 48)), be.zeros((64, 1))
        y, act, probe = be.empty((64, 32)), be.empty((64, 32)), be.empty((64, 32))
        launches = []
        for step in range(3):
            before = be.plan_stats["launches"] if hasattr(be, "plan_stats") and be.plan_stats else 0
            if block:
                be.begin(Block.minibatch, step)
            be.compound_dot(w, x, y)
            y[:] = y + b                       # bias ...
            act[:] = be.maximum(y, 0) + 0.1 * be.minimum(y, 0)      # ... and activation: one kernel
            probe[:] = act * 2.0
            seen = probe.get()                 # a host read inside the block sees all of it
            vw[:] = 0.9 * vw - 0.01 * gw
            w[:] = w + vw
            vb[:] = 0.9 * vb - 0.01 * gb
            b[:] = b + vb
            if block:
                be.end(Block.minibatch, step)
            if hasattr(be, "plan_stats") and be.plan_stats:
                launches.append(be.plan_stats["launches"] - before)
        return [t.get() for t in (w, b, vw, vb, act)] + [seen], launches

    cpu, hip = pair
    want, _ = program(cpu, True)
    plain, n_plain = program(hip, False)
    fused, n_fused = program(hip, True)
    for a, b_, c in zip(want, plain, fused):
        assert_close(b_, a, rtol=1e-5, atol=1e-6, what="outside a block")
        assert_close(c, a, rtol=1e-5, atol=1e-6, what="inside a minibatch block")
    # three elementwise statements after the product fuse into one launch, the four update
    # statements into two (two shapes): 7 statements, 3 kernels
    assert n_plain[-1] == 7 and n_fused[-1] == 3, (n_plain, n_fused)


@pytest.mark.gpu
def test_vectors_read_inside_a_group_must_not_live_in_a_tensor_the_group_writes(pair):
    """row / column vectors are read by lanes other than the ones that would
    write them: a statement whose vector operand is a row of another
    statement's output does not join that statement's group"""
    rs = np.random.RandomState(12)
    a0, b0 = rs.standard_normal((40, 96)).astype(np.float32), rs.standard_normal((40, 96)).astype(np.float32)
    r0, c0 = rs.standard_normal((1, 96)).astype(np.float32), rs.standard_normal((40, 1)).astype(np.float32)
    res, counts = [], []
    for be in pair:
        a, b, row, col = be.array(a0), be.array(b0), be.array(r0), be.array(c0)
        out1, out2 = be.empty((40, 96)), be.empty((40, 96))
        n0 = be.plan_stats["launches"] if getattr(be, "plan_stats", None) else 0
        with be.fused() if hasattr(be, "fused") else _Null():
            out1[:] = a * row + col                 # independent vectors: these two share a kernel
            out2[:] = out1 - b * col
        n1 = be.plan_stats["launches"] if getattr(be, "plan_stats", None) else 0
        with be.fused() if hasattr(be, "fused") else _Null():
            a[:] = a + 1.0                          # writes a ...
            out2[:] = b + a[3:4, :]                 # ... whose row 3 every lane of this statement reads
        n2 = be.plan_stats["launches"] if getattr(be, "plan_stats", None) else 0
        res.append([t.get() for t in (out1, out2, a)])
        counts.append((n1 - n0, n2 - n1))
    for w, g in zip(*res):
        assert_close(g, w, rtol=1e-5, atol=1e-6)
    assert counts[1] == (1, 2)


class _Null(object):
    def __enter__(self):
        return self

    def __exit__(self, *exc):
        return False


@pytest.mark.gpu
def test_a_stretch_that_falls_into_several_groups_is_replayed_as_one_recording(hip):
    """two shapes and a reduction between elementwise statements: the stretch runs
    as four groups; from the second identical minibatch on it is served by ONE
    keyed lookup (a split recording under the stretch's key), with the numbers
    of every group re-bound -- results against numpy for five steps with a
    step-dependent rate"""
    from neon_amd.backends.backend import Block
    from neon_amd.backends.nervanahip import _RecordedSplit
    be = hip
    rs = np.random.RandomState(21)
    w0, g0 = rs.standard_normal((96, 40)).astype(np.float32), rs.standard_normal((96, 40)).astype(np.float32)
    b0, h0 = rs.standard_normal((96, 1)).astype(np.float32), rs.standard_normal((96, 1)).astype(np.float32)
    w, g, b, h = be.array(w0), be.array(g0), be.array(b0), be.array(h0)
    norm, out = be.empty((96, 1)), be.empty((96, 40))
    wn, bn = w0.copy(), b0.copy()
    for step in range(5):
        lr = np.float32(0.1 / (step + 1))
        replayed = be.plan_stats["replayed"]
        be.begin(Block.minibatch, step)
        w[:] = w - float(lr) * g                 # shape (96,40)
        b[:] = b - float(lr) * h                 # shape (96,1): another group
        norm[:] = be.sum(w * w, axis=1)          # a reduction: a group of its own
        out[:] = w * float(step + 2) + b         # elementwise again
        be.end(Block.minibatch, step)
        wn = wn - lr * g0
        bn = bn - lr * h0
        assert_close(w.get(), wn, rtol=1e-5, atol=1e-6, what="w, step %d" % step)
        assert_close(b.get(), bn, rtol=1e-5, atol=1e-6, what="b, step %d" % step)
        assert_close(norm.get(), (wn * wn).sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-5, what="norm, step %d" % step)
        assert_close(out.get(), wn * np.float32(step + 2) + bn, rtol=1e-5, atol=1e-5, what="out, step %d" % step)
        if step >= 1 and be._replayer is not None:
            # one replay for the whole stretch, not one per group
            assert be.plan_stats["replayed"] - replayed == 1, (step, be.plan_stats["replayed"] - replayed)
    if be._replayer is not None:
        assert any(isinstance(e, _RecordedSplit) and len(e.parts) >= 3 for e in be._launch_cache.values())
