"""Small clients of the backend API used by the tests: the activation, cost,
metric and parameter-update op-trees that neon's layers build, written here
from their formulas (the reference file:line each one states is cited) so the
tests need nothing but the backend itself."""
import numpy as np


# ---- activations (reference neon/transforms/activation.py) ----------------------------
def softmax(be, x):                 # activation.py:216-226
    return be.fprop_softmax(x, 0)


def tanh(be, x):                    # activation.py:271-281
    return be.tanh(x)


def logistic(be, x):                # activation.py:334-344
    return be.sig(x)


def rectlin(be, x, slope=0.0):      # activation.py:73-86
    return be.maximum(x, 0) + slope * be.minimum(0, x)


# ---- costs (reference neon/transforms/cost.py) ----------------------------------------
def cross_entropy_binary(be, y, t):     # cost.py:83-95
    return be.sum(be.safelog(1 - y) * (t - 1) - be.safelog(y) * t, axis=0)


def cross_entropy_multi(be, y, t):      # cost.py:142-159
    return be.sum(-t * be.safelog(y), axis=0)


def sum_squared(be, y, t):              # cost.py:176-189
    return be.sum(be.square(y - t), axis=0) / 2.


def mean_squared(be, y, t):             # cost.py:192-205
    return be.mean(be.square(y - t), axis=0) / 2.


# ---- metrics ----------------------------------------------------------------------------
def misclassification(be, y, t):        # cost.py:409-425
    n = y.shape[1]
    preds, hyps = be.empty((1, n), dtype=np.int32), be.empty((1, n), dtype=np.int32)
    wrong = be.empty((1, n))
    preds[:] = be.argmax(y, axis=0)
    hyps[:] = be.argmax(t, axis=0)
    wrong[:] = be.not_equal(preds, hyps)
    return wrong.get().mean()


def precision_recall(be, y, t, eps=1e-6):       # cost.py:485-517
    k = y.shape[0]
    stats, out = be.empty((k, 3)), be.empty((k, 2))
    stats[:, 0] = be.sum(y * t, axis=1)
    stats[:, 1] = be.sum(y, axis=1)
    stats[:, 2] = be.sum(t, axis=1)
    out[:, 0] = stats[:, 0] / (stats[:, 1] + eps)
    out[:, 1] = stats[:, 0] / (stats[:, 2] + eps)
    return out.get().mean(axis=0)


# ---- parameter updates (reference neon/optimizers/optimizer.py), each run between
#      be.begin(Block.update) / be.end(Block.update) so that a backend may fuse them ------
def _grouped(be, body):
    from neon_amd.backends.backend import Block
    be.begin(Block.update, 0)
    try:
        body()
    finally:
        be.end(Block.update, 0)


def adam_update(be, p, g, m, v, t, lr=1e-3, b1=0.9, b2=0.999, eps=1e-8):       # optimizer.py:907-930
    def body():
        l = lr * be.sqrt(1 - b2 ** t) / (1 - b1 ** t)
        gs = g / be.bsz
        m[:] = m * b1 + (1. - b1) * gs
        v[:] = v * b2 + (1. - b2) * gs * gs
        p[:] = p - (l * m) / (be.sqrt(v) + eps)
    _grouped(be, body)


def momentum_update(be, p, g, vel, lr=0.1, mom=0.9, wdecay=0.0005):             # optimizer.py:499-540
    def body():
        gs = g / be.bsz
        vel[:] = mom * vel - lr * (gs + wdecay * p)
        p[:] = p + vel
    _grouped(be, body)


def rmsprop_update(be, p, g, state, lr=2e-3, decay=0.95, eps=1e-6):             # optimizer.py:603-633
    def body():
        gs = g / be.bsz
        state[:] = decay * state + be.square(gs) * (1.0 - decay)
        p[:] = p - (gs * lr) / (be.sqrt(state + eps) + eps)
    _grouped(be, body)


def adadelta_update(be, p, g, gsq, dsq, delta, decay=0.95, eps=1e-6):           # optimizer.py:796-822
    def body():
        gs = g / be.bsz
        gsq[:] = gsq * decay + (1. - decay) * gs * gs
        delta[:] = be.sqrt((dsq + eps) / (gsq + eps)) * gs
        dsq[:] = dsq * decay + (1. - decay) * delta * delta
        p[:] = p - delta
    _grouped(be, body)
