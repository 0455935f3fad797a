"""The callers together: a two-layer perceptron trained with nothing but the
backend's tensor API -- compound_dot for the products, activation / cost
op-trees, fused optimizer updates -- on the oracle and on the hip backend from
the same initial values.  The loss falls and both backends follow the same
trajectory."""
import numpy as np
import pytest

from neon_amd.optimizers import Adam, GradientDescentMomentum
from neon_amd.transforms import CrossEntropyMulti, Softmax, Tanh
from utils import assert_close

NIN, NHID, NOUT, BATCH = 48, 64, 10, 128


class Dense(object):
    def __init__(self, be, w):
        self.be = be
        self.W = be.array(w)
        self.dW = be.zeros(w.shape)
        self.states = []

    def get_params(self):
        return ((self.W, self.dW), self.states)


def _train(be, make_opt, steps, seed=0):
    rs = np.random.RandomState(seed)
    x = rs.standard_normal((NIN, BATCH)).astype(np.float32)
    labels = rs.randint(0, NOUT, size=BATCH)
    t = np.zeros((NOUT, BATCH), np.float32)
    t[labels, np.arange(BATCH)] = 1
    l1 = Dense(be, (rs.standard_normal((NHID, NIN)) * 0.1).astype(np.float32))
    l2 = Dense(be, (rs.standard_normal((NOUT, NHID)) * 0.1).astype(np.float32))
    act, out_act, cost, opt = Tanh(), Softmax(), CrossEntropyMulti(), make_opt()
    for obj in (act, out_act, cost, opt):
        obj.be = be
    old_bsz, be.bsz = be.bsz, BATCH
    X, T = be.array(x), be.array(t)
    pre1, h = be.empty((NHID, BATCH)), be.empty((NHID, BATCH))
    pre2, y = be.empty((NOUT, BATCH)), be.empty((NOUT, BATCH))
    d2, d1 = be.empty((NOUT, BATCH)), be.empty((NHID, BATCH))
    loss = be.empty((1, 1))
    losses = []
    try:
        for step in range(steps):
            be.compound_dot(l1.W, X, pre1)
            h[:] = act(pre1)
            be.compound_dot(l2.W, h, pre2)
            y[:] = out_act(pre2)
            loss[:] = be.sum(cost(y, T), axis=1) / BATCH
            losses.append(float(loss.get()[0, 0]))
            d2[:] = cost.bprop(y, T) * out_act.bprop(pre2)          # softmax + cross-entropy shortcut
            be.compound_dot(d2, h.T, l2.dW)
            be.compound_dot(l2.W.T, d2, d1)
            d1[:] = d1 * act.bprop(h)
            be.compound_dot(d1, X.T, l1.dW)
            opt.optimize([l1, l2], epoch=0)
    finally:
        be.bsz = old_bsz
    return losses, l1.W.get(), l2.W.get()


def test_loss_falls_on_the_oracle(cpu):
    losses, _, _ = _train(cpu, lambda: Adam(learning_rate=0.01), 40)
    assert losses[0] > 2.0 and losses[-1] < 0.5 * losses[0]
    assert all(b < a + 1e-3 for a, b in zip(losses, losses[1:]))


@pytest.mark.gpu
@pytest.mark.parametrize("make_opt", [lambda: Adam(learning_rate=0.01),
                                      lambda: GradientDescentMomentum(0.5, 0.9, wdecay=1e-4, nesterov=True)],
                         ids=["adam", "nesterov"])
def test_hip_follows_the_oracle(pair, make_opt):
    cpu, hip = pair
    lc, w1c, w2c = _train(cpu, make_opt, 25)
    lh, w1h, w2h = _train(hip, make_opt, 25)
    assert lh[-1] < 0.7 * lh[0]
    assert_close(np.array(lh), np.array(lc), rtol=2e-4, atol=1e-5)
    # 25 steps of accumulated rounding differences between two fp32 pipelines
    assert_close(w1h, w1c, rtol=5e-3, atol=5e-4)
    assert_close(w2h, w2c, rtol=5e-3, atol=5e-4)
