"""Recurrent and LSTM layers (neon_amd/layers/recurrent.py) against an
independent float64 numpy forward pass; gradients against central differences
of that forward pass (every weight, every input element), so the layers'
back-propagation through time is checked without restating it.  On the GPU the
same layers are compared with the oracle backend."""
import contextlib

import numpy as np
import pytest

from neon_amd import NervanaObject
from neon_amd.initializers import Array
from neon_amd.layers import GRU, LSTM, Recurrent, RecurrentLast, RecurrentMean, RecurrentSum, Sequential
from neon_amd.transforms import Logistic, Tanh

NIN, NOUT, STEPS, BSZ = 5, 6, 4, 3
NGATES = {"rnn": 1, "lstm": 4, "gru": 3}


@contextlib.contextmanager
def using(be, bsz):
    old, old_bsz = NervanaObject.be, be.bsz
    NervanaObject.be, be.bsz = be, bsz
    try:
        yield be
    finally:
        NervanaObject.be, be.bsz = old, old_bsz


def _sig(z):
    return 1.0 / (1.0 + np.exp(-z))


def _forward64(kind, W, x, proj):
    """loss = sum(proj * outputs) of the layer with packed parameters W
    ((nin + nout + 1, ngates * nout), the layer's own layout) in float64"""
    ng = NGATES[kind]
    g_nout = ng * NOUT
    W_in = W[:NIN].reshape(g_nout, NIN)
    W_rec = W[NIN:-1].reshape(g_nout, NOUT)
    b = W[-1:].reshape(g_nout, 1)
    h, c = np.zeros((NOUT, BSZ)), np.zeros((NOUT, BSZ))
    outs = []
    for s in range(STEPS):
        xs = x[:, s * BSZ:(s + 1) * BSZ]
        if kind == "gru":
            zx = W_in @ xs + b
            rz = _sig(zx[:2 * NOUT] + W_rec[:2 * NOUT] @ h)
            r, u = rz[:NOUT], rz[NOUT:]
            cand = np.tanh(zx[2 * NOUT:] + W_rec[2 * NOUT:] @ (r * h))
            h = (1 - u) * h + u * cand
            outs.append(h)
            continue
        z = W_in @ xs + W_rec @ h + b
        if kind == "rnn":
            h = np.tanh(z)
        else:
            i, f, o = _sig(z[:NOUT]), _sig(z[NOUT:2 * NOUT]), _sig(z[2 * NOUT:3 * NOUT])
            g = np.tanh(z[3 * NOUT:])
            c = f * c + i * g
            h = o * np.tanh(c)
        outs.append(h)
    out = np.concatenate(outs, axis=1)
    return float((proj * out).sum()), out


def _numeric_grad(f, a, eps=1e-6):
    g = np.zeros_like(a)
    flat, gf = a.reshape(-1), g.reshape(-1)
    for k in range(flat.size):
        old = flat[k]
        flat[k] = old + eps
        up = f()
        flat[k] = old - eps
        down = f()
        flat[k] = old
        gf[k] = (up - down) / (2 * eps)
    return g


def _make(be, kind, W):
    nrows = NIN + NOUT + 1
    ng = NGATES[kind]
    init = Array(np.zeros((NOUT, NIN), np.float32))         # placeholder: the packed W is set below
    if kind in ("lstm", "gru"):
        layer = (LSTM if kind == "lstm" else GRU)(NOUT, init, init_inner=Array(np.zeros((NOUT, NOUT), np.float32)),
                                                  activation=Tanh(), gate_activation=Logistic())
    else:
        layer = Recurrent(NOUT, init, init_inner=Array(np.zeros((NOUT, NOUT), np.float32)), activation=Tanh())
    layer.configure((NIN, STEPS))
    layer.prev_layer = True                                  # so that it owns an input-delta buffer
    layer.allocate()
    from neon_amd.layers import DeltasTree
    tree = DeltasTree()
    layer.allocate_deltas(tree)
    tree.allocate_buffers()
    layer.set_deltas(tree)
    assert layer.W.shape == (nrows, ng * NOUT)
    layer.W[:] = W.astype(np.float32)
    return layer


def _check_layer(be, kind, rtol):
    with using(be, BSZ):
        rs = np.random.RandomState(5 + NGATES[kind])
        ng = NGATES[kind]
        W = rs.uniform(-0.6, 0.6, (NIN + NOUT + 1, ng * NOUT))
        x = rs.uniform(-1, 1, (NIN, STEPS * BSZ))
        proj = rs.uniform(-1, 1, (NOUT, STEPS * BSZ))
        layer = _make(be, kind, W)
        W32, x32 = W.astype(np.float32).astype(np.float64), x.astype(np.float32).astype(np.float64)
        out = layer.fprop(be.array(x.astype(np.float32)))
        _, want_out = _forward64(kind, W32, x32, proj)
        assert np.allclose(out.get(), want_out, rtol=1e-5, atol=1e-6)
        deltas = layer.bprop(be.array(proj.astype(np.float32)))
        p32 = proj.astype(np.float32).astype(np.float64)
        gW = _numeric_grad(lambda: _forward64(kind, W32, x32, p32)[0], W32)
        gx = _numeric_grad(lambda: _forward64(kind, W32, x32, p32)[0], x32)
        assert np.abs(layer.dW.get() - gW).max() < rtol * np.abs(gW).max()
        assert np.abs(deltas.get() - gx).max() < rtol * np.abs(gx).max()
        # a second pass over the same input gives the same result (state buffers are re-used, not accumulated)
        out2 = layer.fprop(be.array(x.astype(np.float32)))
        assert np.allclose(out2.get(), want_out, rtol=1e-5, atol=1e-6)
        return out.get(), layer.dW.get(), deltas.get()


@pytest.mark.parametrize("kind", ["rnn", "lstm", "gru"])
def test_recurrent_layers_against_float64_and_finite_differences(cpu, kind):
    _check_layer(cpu, kind, 2e-4)


def test_recurrent_output_layers(cpu):
    with using(cpu, BSZ):
        rs = np.random.RandomState(2)
        x = rs.uniform(-1, 1, (NOUT, STEPS * BSZ)).astype(np.float32)
        err = rs.uniform(-1, 1, (NOUT, BSZ)).astype(np.float32)
        steps = [x[:, s * BSZ:(s + 1) * BSZ] for s in range(STEPS)]
        for cls, want, back in ((RecurrentSum, sum(steps), [err] * STEPS),
                                (RecurrentMean, sum(steps) / STEPS, [err / STEPS] * STEPS),
                                (RecurrentLast, steps[-1], [0 * err] * (STEPS - 1) + [err])):
            from neon_amd.layers import DeltasTree
            layer = cls()
            layer.configure((NOUT, STEPS))
            layer.prev_layer = True
            layer.allocate()
            tree = DeltasTree()
            layer.allocate_deltas(tree)
            tree.allocate_buffers()
            layer.set_deltas(tree)
            out = layer.fprop(cpu.array(x))
            assert np.allclose(out.get(), want, atol=1e-6), cls.__name__
            deltas = layer.bprop(cpu.array(err))
            assert np.allclose(deltas.get(), np.concatenate(back, axis=1), atol=1e-6), cls.__name__


def _check_unroll(be, reverse):
    """compound_rnn_unroll_fprop / bprop against a float64 loop: forward over
    the steps (or backward, for the reverse direction of a bidirectional
    layer), and the back-propagated deltas of the same loop"""
    rs = np.random.RandomState(11 + reverse)
    Wr = rs.uniform(-0.6, 0.6, (NOUT, NOUT)).astype(np.float32)
    b = rs.uniform(-0.5, 0.5, (NOUT, 1)).astype(np.float32)
    ff = rs.uniform(-1, 1, (NOUT, STEPS * BSZ)).astype(np.float32)
    err = rs.uniform(-1, 1, (NOUT, STEPS * BSZ)).astype(np.float32)
    used = STEPS - 1
    order = list(range(used))[::-1] if reverse else list(range(used))
    sl = [slice(t * BSZ, (t + 1) * BSZ) for t in range(STEPS)]
    h64 = np.zeros((NOUT, STEPS * BSZ))
    prev = np.zeros((NOUT, BSZ))
    for t in order:
        h64[:, sl[t]] = np.tanh(Wr.astype(np.float64) @ prev + ff[:, sl[t]] + b)
        prev = h64[:, sl[t]]
    d64 = err.astype(np.float64).copy()
    for t in order[::-1]:
        d64[:, sl[t]] *= 1 - h64[:, sl[t]] ** 2
        src = order[order.index(t) - 1] if order.index(t) > 0 else None
        if src is not None:
            d64[:, sl[src]] += Wr.T.astype(np.float64) @ d64[:, sl[t]]
    with using(be, BSZ):
        act = Tanh()
        W_d, b_d = be.array(Wr), be.array(b)
        zero = be.zeros((NOUT, BSZ))
        for shared in (False, True):
            h_buf = be.array(ff) if shared else be.zeros((NOUT, STEPS * BSZ))
            ff_buf = h_buf if shared else be.array(ff)
            h_s = [h_buf[:, s] for s in sl]
            ff_s = h_s if shared else [ff_buf[:, s] for s in sl]
            prev_s = (h_s[1:used] + [zero] * (STEPS - used + 1)) if reverse else ([zero] + h_s[:-1])
            be.compound_rnn_unroll_fprop(W_d, prev_s, ff_s, h_s, b_d, NOUT, STEPS, used, act, reverse)
            got = h_buf.get()
            for t in order:
                assert np.allclose(got[:, sl[t]], h64[:, sl[t]], rtol=1e-5, atol=1e-6), (shared, t)
            if not shared:
                assert not got[:, sl[STEPS - 1]].any()       # the unused step stays untouched
        d_buf = be.array(err)
        d_s = [d_buf[:, s] for s in sl][:used]
        sink = be.zeros((NOUT, BSZ))
        dprev_s = (d_s[1:] + [sink]) if reverse else ([sink] + d_s[:-1])   # d_s holds the used steps only
        be.compound_rnn_unroll_bprop(W_d.T, dprev_s, d_s, h_s, NOUT, STEPS, used, act, not reverse)
        got = d_buf.get()
        for t in order:
            assert np.allclose(got[:, sl[t]], d64[:, sl[t]], rtol=1e-5, atol=1e-6), t
        return h_buf.get(), got


@pytest.mark.parametrize("reverse", [False, True])
def test_rnn_unroll_helpers(cpu, reverse):
    _check_unroll(cpu, reverse)


@pytest.mark.gpu
@pytest.mark.parametrize("reverse", [False, True])
def test_rnn_unroll_helpers_on_hip(pair, reverse):
    cpu, hip = pair
    for g, w in zip(_check_unroll(hip, reverse), _check_unroll(cpu, reverse)):
        assert np.allclose(g, w, rtol=2e-5, atol=2e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("kind", ["rnn", "lstm", "gru"])
def test_recurrent_layers_on_hip(pair, kind):
    cpu, hip = pair
    want = _check_layer(cpu, kind, 2e-4)
    got = _check_layer(hip, kind, 2e-4)
    for g, w in zip(got, want):
        assert np.allclose(g, w, rtol=2e-5, atol=2e-6)
