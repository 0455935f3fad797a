"""
The five benchmark op-trees, written once against the backend API so that the
hip backend, the CPU oracle, the tests and the benchmark all run the very same
expressions on the very same seeded inputs.

Config k draws from ``np.random.RandomState(20240 + k)`` in the order listed in
its ``inputs_*`` function; N(mu, sigma) means ``standard_normal * sigma + mu``.
"""
import numpy as np

SEED_BASE = 20240

C1_SHAPE = (4096, 128)
C2_SHAPE = (1000, 128)
C3_SHAPE = (5000, 5000)
C4_SHAPE = (256, 100352)
C5_SHAPE = (32000, 256)

ADAM = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8)


def _rs(k):
    return np.random.RandomState(SEED_BASE + k)


# ---- inputs (host arrays) ---------------------------------------------------------
def inputs_c1(shape=C1_SHAPE):
    rs = _rs(1)
    x = rs.standard_normal(shape).astype(np.float32)
    y = rs.standard_normal(shape).astype(np.float32)
    return x, y


def inputs_c2(shape=C2_SHAPE):
    rs = _rs(2)
    return ((rs.standard_normal(shape) * 3.0).astype(np.float32),)


def inputs_c3(shape=C3_SHAPE):
    rs = _rs(3)
    grad = (rs.standard_normal(shape) * 1e-2).astype(np.float32)
    param = (rs.standard_normal(shape) * 0.05).astype(np.float32)
    return grad, param


def inputs_c4(shape=C4_SHAPE):
    rs = _rs(4)
    x = (rs.standard_normal(shape) * 2.0 + 0.5).astype(np.float32).astype(np.float16)
    gamma = rs.uniform(0.5, 1.5, (shape[0], 1)).astype(np.float32)
    beta = (rs.standard_normal((shape[0], 1)) * 0.1).astype(np.float32)
    return x, gamma, beta


def inputs_c5(shape=C5_SHAPE):
    rs = _rs(5)
    x = (rs.standard_normal(shape) * 4.0).astype(np.float32)
    idx = rs.randint(0, shape[0], size=(1, shape[1])).astype(np.int32)
    return x, idx


# ---- op-trees -------------------------------------------------------------------------
def c1a(be, out, x, y):
    out[:] = 0.5 * x + 2.0 * y


def c1b(be, out):
    out[:] = be.sig(out)


def c1_fused(be, out, x, y):
    out[:] = be.sig(0.5 * x + 2.0 * y)


def c2_softmax(be, out, x):
    out[:] = be.exp(x - be.max(x, axis=0)) / be.sum(be.exp(x - be.max(x, axis=0)), axis=0)


def c2_softmax_neon(be, out, x):
    """the form the reference's Softmax activation builds (activation.py:216-226)"""
    out[:] = be.fprop_softmax(x, 0)


def c3_adam_step(be, param, grad, m, v, t, lr=ADAM["lr"], beta1=ADAM["beta1"],
                 beta2=ADAM["beta2"], eps=ADAM["eps"]):
    """The body of Adam.optimize (reference optimizer.py:907-930) for one
    parameter tensor, without clipping; ``grad / be.bsz`` with bsz = 1."""
    l = lr * be.sqrt(1 - beta2 ** t) / (1 - beta1 ** t)
    m[:] = m * beta1 + (1. - beta1) * grad
    v[:] = v * beta2 + (1. - beta2) * grad * grad
    param[:] = param - (l * m) / (be.sqrt(v) + eps)


def c4_rownorm(be, out, x, gamma, beta, eps=1e-5):
    """Batch-norm forward as an op-tree (BatchNormAutodiff.get_forward_optree,
    reference layer.py:2592-2600): statistics along axis 1."""
    mean = be.mean(x, axis=1)
    var = be.var(x, axis=1)
    out[:] = gamma * (x - mean) / be.sqrt(var + eps) + beta


def c5a_argmax(be, amax, x):
    amax[:] = be.argmax(x, axis=0)


def c5b_max(be, mx, x):
    mx[:] = be.max(x, axis=0)


def c5c_cross_entropy(be, ce, x, onehot):
    """-sum(onehot * log(softmax(x)), axis 0); ``onehot`` is either a dense 0/1
    tensor or ``be.onehot(idx, axis=0)`` evaluated inside the kernel."""
    sm = be.exp(x - be.max(x, axis=0)) / be.sum(be.exp(x - be.max(x, axis=0)), axis=0)
    ce[:] = -be.sum(onehot * be.log(sm), axis=0)


# ---- algorithmic bytes per launch group (each tensor counted once) ---------------------
def bytes_c1a(shape=C1_SHAPE):
    return 3 * 4 * shape[0] * shape[1]


def bytes_c1b(shape=C1_SHAPE):
    return 2 * 4 * shape[0] * shape[1]


def bytes_c2(shape=C2_SHAPE):
    return 2 * 4 * shape[0] * shape[1]


def bytes_c3(shape=C3_SHAPE, fused=True):
    return (7 if fused else 10) * 4 * shape[0] * shape[1]


def bytes_c4(shape=C4_SHAPE):
    return 2 * 2 * shape[0] * shape[1] + 2 * 4 * shape[0]


def bytes_c5_reduce(shape=C5_SHAPE):
    return 4 * shape[0] * shape[1] + 4 * shape[1]


def bytes_c5c(shape=C5_SHAPE, dense_onehot=False):
    b = 4 * shape[0] * shape[1] + 2 * 4 * shape[1]
    return b + (4 * shape[0] * shape[1] if dense_onehot else 0)
