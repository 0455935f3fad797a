"""Layers and the sequential container (neon_amd/layers).

On the oracle backend a batch-normalised, dropped-out two-block perceptron is
held against an independent float64 numpy evaluation of the same network and
its hand-derived gradients (outputs, cost, every parameter gradient); the
embedding layer against numpy indexing and a scatter-add.  On the GPU the same
network is trained for a few optimizer steps on both backends from the same
values and the trajectories are compared."""
import contextlib

import numpy as np
import pytest

from neon_amd import NervanaObject
from neon_amd.initializers import Array, Constant
from neon_amd.layers import (Activation, Affine, BatchNorm, Bias, Dropout, GeneralizedCost, Linear, LookupTable,
                             Sequential, interpret_in_shape)
from neon_amd.optimizers import Adam
from neon_amd.transforms import CrossEntropyMulti, Rectlin, Softmax, Tanh
from utils import assert_close

NIN, NHID, NOUT, BATCH = 24, 40, 10, 64


@contextlib.contextmanager
def using(be, bsz):
    old, old_bsz = NervanaObject.be, be.bsz
    NervanaObject.be, be.bsz = be, bsz
    try:
        yield be
    finally:
        NervanaObject.be, be.bsz = old, old_bsz


def _values(seed=3):
    rs = np.random.RandomState(seed)
    x = rs.standard_normal((NIN, BATCH)).astype(np.float32)
    labels = rs.randint(0, NOUT, size=BATCH)
    t = np.zeros((NOUT, BATCH), np.float32)
    t[labels, np.arange(BATCH)] = 1
    w1 = (rs.standard_normal((NHID, NIN)) * 0.3).astype(np.float32)
    w2 = (rs.standard_normal((NOUT, NHID)) * 0.3).astype(np.float32)
    return x, t, w1, w2


def _build(be, w1, w2, keep=0.7):
    layers = [Affine(NHID, Array(w1), batch_norm=True, activation=Tanh()),
              Dropout(keep=keep),
              Affine(NOUT, Array(w2), bias=Constant(0.1), activation=Softmax())]
    net = Sequential(layers)
    net.configure((NIN, 1))
    net.allocate()
    net.allocate_deltas()
    cost = GeneralizedCost(CrossEntropyMulti())
    cost.initialize(net)
    return net, cost


def test_shapes_and_ownership(cpu):
    assert interpret_in_shape(5) == (5, 1) and interpret_in_shape((5, 3)) == (5, 3)
    assert interpret_in_shape((3, 4, 4)) == (48, 1)
    with using(cpu, BATCH):
        x, t, w1, w2 = _values()
        net, cost = _build(cpu, w1, w2)
        kinds = [type(layer) for layer in net.layers]
        assert kinds == [Linear, BatchNorm, Activation, Dropout, Linear, Bias, Activation]
        lin1, bn, act1, drop, lin2, bias, act2 = net.layers
        assert lin1.outputs.shape == (NHID, BATCH) and lin2.outputs.shape == (NOUT, BATCH)
        assert lin1.deltas is None                         # nothing below the first layer
        assert bn.xsum is lin1.batch_sum and not bn.compute_batch_sum
        # delta-owning layers alternate between the container's two buffers
        owners = [layer for layer in net.layers if layer.deltas is not None]
        assert [type(o) for o in owners] == [BatchNorm, Activation, Linear, Activation]
        bases = [o.deltas.base if o.deltas.base is not None else o.deltas for o in owners]
        assert bases[0] is not bases[1] and bases[0] is bases[2] and bases[1] is bases[3]
        assert [type(layer) for layer in net.layers_to_optimize] == [Linear, BatchNorm, Linear, Bias]
        with pytest.raises(AttributeError):
            Affine(4, Constant(0), bias=Constant(0), batch_norm=True)


def _float64_network(x, t, w1, w2, mask, eps=1e-3, bias=0.1):
    """forward and hand-derived backward of the network of _build, in float64"""
    x, t, w1, w2, mask = (a.astype(np.float64) for a in (x, t, w1, w2, mask))
    B = x.shape[1]
    z1 = w1 @ x
    mean, var = z1.mean(axis=1, keepdims=True), z1.var(axis=1, keepdims=True)
    xhat = (z1 - mean) / np.sqrt(var + eps)
    a1 = np.tanh(xhat)                                      # gamma = 1, beta = 0
    d = mask * a1
    z2 = w2 @ d + bias
    e = np.exp(z2 - z2.max(axis=0))
    p = e / e.sum(axis=0)
    cost = np.mean(-np.sum(t * np.log(p), axis=0))
    dz2 = p - t
    g = {"db2": dz2.sum(axis=1, keepdims=True), "dW2": dz2 @ d.T}
    dy1 = mask * (w2.T @ dz2) * (1 - a1 * a1)
    g["dgamma"] = (dy1 * xhat).sum(axis=1, keepdims=True)
    g["dbeta"] = dy1.sum(axis=1, keepdims=True)
    dz1 = (dy1 - (xhat * g["dgamma"] + g["dbeta"]) / B) / np.sqrt(var + eps)
    g["dW1"] = dz1 @ x.T
    return p, cost, g


def test_network_matches_float64_model(cpu):
    with using(cpu, BATCH):
        x, t, w1, w2 = _values()
        net, cost = _build(cpu, w1, w2)
        X, T = cpu.array(x), cpu.array(t)
        out = net.fprop(X)
        c = cost.get_cost(out, T)
        net.bprop(cost.get_errors(out, T))
        lin1, bn, act1, drop, lin2, bias, act2 = net.layers
        mask = drop.keep_mask.get()
        assert set(np.unique(mask)) <= {0.0, 1.0} and 0.5 < mask.mean() < 0.9
        p, want_cost, g = _float64_network(x, t, w1, w2, mask)
        assert_close(out.get(), p, rtol=1e-4, atol=1e-6, what="softmax output")
        assert abs(float(c[0, 0]) - want_cost) < 1e-4 * want_cost
        for name, got in (("dW2", lin2.dW), ("db2", bias.dW), ("dgamma", bn.grad_gamma),
                          ("dbeta", bn.grad_beta), ("dW1", lin1.dW)):
            scale = np.abs(g[name]).max()
            assert np.abs(got.get() - g[name]).max() < 2e-4 * scale, name
        # inference: dropout scales by keep, batch norm uses its running statistics
        out_inf = net.fprop(X, inference=True).get()
        assert np.allclose(out_inf.sum(axis=0), 1.0, atol=1e-5)


def test_lookup_table_layer(cpu):
    vocab, dim, nin, bsz = 50, 8, 5, 16
    with using(cpu, bsz):
        rs = np.random.RandomState(1)
        table = rs.standard_normal((vocab, dim)).astype(np.float32)
        ids = rs.randint(0, vocab, size=(nin, bsz)).astype(np.int32)
        layer = LookupTable(vocab, dim, Array(table), pad_idx=0)
        layer.configure((nin, 1))
        layer.allocate()
        table[0] = 0                                        # the padding row is cleared
        out = layer.fprop(cpu.array(ids, dtype=np.int32)).get()
        flat = ids.reshape(-1)
        assert out.shape == (dim, nin * bsz) and np.array_equal(out, table[flat].T)
        err = rs.standard_normal((dim, nin * bsz)).astype(np.float32)
        layer.bprop(cpu.array(err))
        want = np.zeros((vocab, dim))
        np.add.at(want, flat, err.T.astype(np.float64))
        want[0] = 0
        assert np.allclose(layer.dW.get(), want, rtol=1e-5, atol=1e-5)


def _train(be, steps):
    with using(be, BATCH):
        x, t, w1, w2 = _values()
        be.rng_reset()
        net, cost = _build(be, w1, w2, keep=1.0)            # device and host masks differ by construction
        opt = Adam(learning_rate=0.01)
        X, T = be.array(x), be.array(t)
        costs = []
        for _ in range(steps):
            out = net.fprop(X)
            costs.append(float(cost.get_cost(out, T)[0, 0]))
            net.bprop(cost.get_errors(out, T))
            opt.optimize(net.layers_to_optimize, epoch=0)
        params = [p.get() for layer in net.layers_to_optimize
                  for (p, _), _ in (layer.get_params() if isinstance(layer.get_params(), list)
                                    else [layer.get_params()])]
        return costs, params


def test_training_lowers_the_cost_on_the_oracle(cpu):
    costs, _ = _train(cpu, 15)
    assert costs[-1] < 0.6 * costs[0]


@pytest.mark.gpu
def test_hip_trains_like_the_oracle(pair):
    cpu, hip = pair
    want_costs, want_params = _train(cpu, 8)
    got_costs, got_params = _train(hip, 8)
    assert np.allclose(got_costs, want_costs, rtol=2e-4)
    for got, want in zip(got_params, want_params):
        assert_close(got, want, rtol=2e-3, atol=2e-4, what="parameters after 8 Adam steps")


@pytest.mark.gpu
def test_hip_layers_match_float64_model(hip):
    with using(hip, BATCH):
        x, t, w1, w2 = _values()
        net, cost = _build(hip, w1, w2)
        X, T = hip.array(x), hip.array(t)
        out = net.fprop(X)
        c = cost.get_cost(out, T)
        net.bprop(cost.get_errors(out, T))
        lin1, bn, act1, drop, lin2, bias, act2 = net.layers
        mask = drop.keep_mask.get()
        p, want_cost, g = _float64_network(x, t, w1, w2, mask)
        assert_close(out.get(), p, rtol=1e-4, atol=1e-6, what="softmax output")
        assert abs(float(c[0, 0]) - want_cost) < 1e-4 * want_cost
        for name, got in (("dW2", lin2.dW), ("db2", bias.dW), ("dgamma", bn.grad_gamma),
                          ("dbeta", bn.grad_beta), ("dW1", lin1.dW)):
            scale = np.abs(g[name]).max()
            assert np.abs(got.get() - g[name]).max() < 2e-4 * scale, name
