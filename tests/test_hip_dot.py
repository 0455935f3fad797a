"""Dense contraction hand-off: compound_dot and `dot` nodes inside op-trees.

The product itself is the library GEMM's; what is checked here is the operand
plumbing (transposed views, strided views, leading dimensions), the alpha /
beta / ReLU / row-sum epilogues and the staging of `dot` nodes through
temporaries -- against the oracle backend and a float64 numpy product.
"""
import numpy as np
import pytest

from neon_amd.backends.autodiff import Autodiff
from utils import assert_close


def _rand(rs, shape, dtype=np.float32):
    return (-1 + 2 * rs.rand(*shape)).astype(dtype)


def _want(a, b, c, alpha, beta, relu):
    prod = alpha * (a.astype(np.float64) @ b.astype(np.float64))
    if relu:
        prod = np.maximum(prod, 0)
    return prod + beta * c.astype(np.float64)


CASES = [
    # m, n, k, transA, transB, alpha, beta, relu
    (64, 48, 32, False, False, 1.0, 0.0, False),
    (65, 47, 33, True, False, 1.0, 0.0, False),
    (65, 47, 33, False, True, 1.0, 0.0, False),
    (128, 256, 512, False, False, 0.5, 0.0, False),
    (128, 256, 512, True, False, 2.0, 0.75, False),
    (100, 30, 70, False, True, 1.5, -0.5, True),
    (100, 30, 70, False, False, 1.0, 0.0, True),
    (1, 40, 50, False, False, 1.0, 0.0, False),
    (40, 1, 50, False, False, 1.0, 1.0, False),
    (40, 1, 50, True, False, 1.0, 0.0, False),
    (7, 9, 1, False, False, 1.0, 0.0, False),
]


def test_compound_dot_oracle(cpu):
    rs = np.random.RandomState(0)
    for m, n, k, ta, tb, alpha, beta, relu in CASES:
        a = _rand(rs, (k, m) if ta else (m, k))
        b = _rand(rs, (n, k) if tb else (k, n))
        c = _rand(rs, (m, n))
        A, B, C = cpu.array(a), cpu.array(b), cpu.array(c)
        bsum = cpu.empty((m, 1))
        cpu.compound_dot(A.T if ta else A, B.T if tb else B, C, alpha=alpha, beta=beta, relu=relu, bsum=bsum)
        want = _want(a.T if ta else a, b.T if tb else b, c, alpha, beta, relu)
        assert_close(C.get(), want.astype(np.float32), rtol=1e-4, atol=1e-4 * k)
        assert_close(bsum.get(), want.sum(axis=1, keepdims=True).astype(np.float32), rtol=1e-4, atol=1e-4 * k * n)


def test_dot_gradients_oracle(cpu):
    """d sum(A.B * E) / dA = E.B^T and / dB = A^T.E"""
    rs = np.random.RandomState(1)
    a, b, e = _rand(rs, (6, 5)), _rand(rs, (5, 7)), _rand(rs, (6, 7))
    A, B = cpu.array(a), cpu.array(b)
    ga, gb = Autodiff(cpu.dot(A, B), cpu, next_error=cpu.array(e)).get_grad_asnumpyarray([A, B])
    assert_close(ga, e @ b.T, rtol=1e-5, atol=1e-5)
    assert_close(gb, a.T @ e, rtol=1e-5, atol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,tol", [(np.float32, 1e-5), (np.float16, 2e-3)], ids=["f32", "f16"])
@pytest.mark.parametrize("case", CASES, ids=[str(i) for i in range(len(CASES))])
def test_compound_dot_hip(hip, case, dtype, tol):
    m, n, k, ta, tb, alpha, beta, relu = case
    rs = np.random.RandomState(m * 7 + n)
    a = _rand(rs, (k, m) if ta else (m, k), dtype)
    b = _rand(rs, (n, k) if tb else (k, n), dtype)
    c = _rand(rs, (m, n), dtype)
    A, B, C = hip.array(a, dtype=dtype), hip.array(b, dtype=dtype), hip.array(c, dtype=dtype)
    bsum = hip.empty((m, 1), dtype=np.float32)
    out = hip.compound_dot(A.T if ta else A, B.T if tb else B, C, alpha=alpha, beta=beta, relu=relu, bsum=bsum)
    assert out is C
    want = _want(a.T if ta else a, b.T if tb else b, c, alpha, beta, relu)
    scale = max(1.0, np.abs(want).max())
    got = C.get()
    assert_close(got, want.astype(dtype), rtol=tol, atol=tol * scale)
    # the row sums are those of the stored C
    assert_close(bsum.get(), got.astype(np.float64).sum(axis=1, keepdims=True).astype(np.float32),
                 rtol=1e-5, atol=1e-5 * scale * n)


@pytest.mark.gpu
def test_compound_dot_views_hip(pair):
    cpu, hip = pair
    rs = np.random.RandomState(5)
    a, b, c = _rand(rs, (96, 80)), _rand(rs, (80, 72)), _rand(rs, (96, 100))
    res = []
    for be in pair:
        A, B, C = be.array(a), be.array(b), be.array(c)
        # row/column windows of the operands, a column window of the output
        be.compound_dot(A[8:72, 16:64], B[16:64, 4:44], C[8:72, 30:70], alpha=1.0, beta=0.5)
        # every second row of A: read in place with a doubled leading dimension
        be.compound_dot(A[0:64:2, :], B, C[0:32, 0:72])
        res.append(C.get())
    assert_close(res[1], res[0], rtol=1e-5, atol=1e-5 * 80)
    assert np.array_equal(res[1][72:, :], c[72:, :])


@pytest.mark.gpu
def test_compound_dot_operands_staged_through_a_copy(pair):
    """operands the GEMM cannot read in place: a view strided along both
    dimensions and a gather view (rows picked by an index tensor)"""
    cpu, hip = pair
    rs = np.random.RandomState(6)
    a, b = _rand(rs, (96, 80)), _rand(rs, (80, 72))
    rows = rs.randint(0, 96, size=(1, 40)).astype(np.int32)
    res = []
    for be in pair:
        A, B = be.array(a), be.array(b)
        C1, C2, C3 = be.zeros((48, 72)), be.zeros((40, 72)), be.zeros((96, 36))
        be.compound_dot(A[0:96:2, 0:80:2], B[0:40, :], C1)
        be.compound_dot(A.take(be.array(rows, dtype=np.int32), axis=0), B, C2)
        be.compound_dot(A, B[:, 0:72:2], C3)
        res.append((C1.get(), C2.get(), C3.get()))
    want = (a[0:96:2, 0:80:2].astype(np.float64) @ b[0:40], a[rows[0]].astype(np.float64) @ b,
            a.astype(np.float64) @ b[:, 0:72:2])
    for got, oracle, w in zip(res[1], res[0], want):
        assert_close(got, w, rtol=1e-5, atol=1e-5 * 80)
        assert_close(got, oracle, rtol=1e-5, atol=1e-5 * 80)


@pytest.mark.gpu
def test_compound_dot_rejects_bad_operands(hip):
    A, B, C = hip.zeros((4, 5)), hip.zeros((6, 3)), hip.zeros((4, 3))
    with pytest.raises(AssertionError):
        hip.compound_dot(A, B, C)
    with pytest.raises(AssertionError):
        hip.compound_dot(hip.zeros((4, 6), dtype=np.float16), B, C)


def _func_dot(be, x0, x1, x2, x3, x4):
    # reference tests/test_backend_autodiff.py Funcs.func_dot
    return (x0 + x3) + be.dot(x1, x2) - (x1 - x2) - be.dot(x3, x4)


def _func_dot_reduction_mix(be, x0, x1, x2, x3, x4):
    # reference tests/test_backend_autodiff.py Funcs.func_dot_reduction_mix
    f1 = be.max(x0, axis=1, keepdims=True)
    f2 = be.min(x1, axis=0, keepdims=True)
    f3 = be.dot(1. / x3, x2 + x4)
    f4 = be.min(x3, axis=0, keepdims=True)
    return f1 + f2 + f3 + f4


@pytest.mark.gpu
@pytest.mark.parametrize("f", [_func_dot, _func_dot_reduction_mix], ids=["dot", "dot_reduction_mix"])
@pytest.mark.parametrize("dim", [2, 48])
def test_dot_in_optree_hip(pair, f, dim):
    rs = np.random.RandomState(dim)
    arrays = [(0.5 + rs.rand(dim, dim)).astype(np.float32) for _ in range(5)]
    vals, grads = [], []
    for be in pair:
        tensors = [be.array(a) for a in arrays]
        out = be.empty((dim, dim))
        for _ in range(2):                       # second pass: nothing stale is replayed
            out[:] = f(be, *tensors)
        vals.append(out.get())
        ad = Autodiff(f(be, *tensors), be)
        grads.append(ad.get_grad_asnumpyarray(tensors))
    assert_close(vals[1], vals[0], rtol=1e-5, atol=1e-5 * dim)
    for g, w in zip(grads[1], grads[0]):
        assert_close(g, w, rtol=1e-4, atol=1e-4 * max(1.0, np.abs(w).max()))


@pytest.mark.gpu
def test_dot_tree_sees_new_values_on_second_run(hip):
    rs = np.random.RandomState(3)
    a, b = _rand(rs, (32, 16)), _rand(rs, (16, 24))
    A, B, out = hip.array(a), hip.array(b), hip.empty((32, 24))
    out[:] = hip.dot(A, B) + 1.0
    A[:] = A * 2.0
    out[:] = hip.dot(A, B) + 1.0
    assert_close(out.get(), (2 * a.astype(np.float64) @ b + 1.0).astype(np.float32), rtol=1e-5, atol=1e-5 * 16)


class _Np(object):
    """numpy float64 evaluation of the same builders"""
    dot = staticmethod(np.dot)

    @staticmethod
    def var(a, axis=None, keepdims=True):
        return np.var(a, axis=axis, keepdims=True)

    @staticmethod
    def std(a, axis=None, keepdims=True):
        return np.std(a, axis=axis, keepdims=True)

    @staticmethod
    def max(a, axis=None, keepdims=True):
        return np.max(a, axis=axis, keepdims=True)

    @staticmethod
    def min(a, axis=None, keepdims=True):
        return np.min(a, axis=axis, keepdims=True)


def _compound_mix(be, x0, x1, x2, x3, x4):
    # reference tests/test_backend_compound_optree.py func_dot_reduction_mix
    f1 = be.std(be.var(x0, axis=0, keepdims=True), axis=1, keepdims=True)
    f2 = be.max(x1, axis=0, keepdims=True) + be.min(x1, axis=0, keepdims=True)
    f3 = be.std(x2, keepdims=True)
    f4 = be.dot(1.0 / x3, x4 / x2)
    f5 = be.dot(x3, x4 - x0)
    f6 = be.dot(x2 / f4, f5 + x3)
    return f1 + f2 + f3 + f4 + 1.0 / (be.dot(f5, f6))


def _compound_transpose_mix(be, x0, x1, x2, x3, x4):
    # reference tests/test_backend_compound_optree.py func_dot_reduction_transpose_mix
    f1 = be.std(be.var(x0, axis=0, keepdims=True), axis=1, keepdims=True)
    f2 = be.max(x1, axis=0, keepdims=True) + be.min(x1, axis=0, keepdims=True)
    f3 = be.std(x2, keepdims=True).T
    f4 = be.dot(1.0 / x3, (x4 / x2).T).T
    f5 = be.dot(x3, (x4 - x0).T)
    f6 = be.dot(x2 / f4.T, f5 + x3).T
    return f1 + f2 + f3 + f4 + 1.0 / (be.dot(f5, f6))


def _compound_inputs(flag, dim):
    rs = np.random.RandomState(17)
    lo, hi = {"pos_rand": (0.5, 1.5), "neg_rand": (-1.5, -0.5), "rand": (0.5, 1.5)}[flag]
    xs = [(lo + (hi - lo) * rs.rand(dim, dim)).astype(np.float32) for _ in range(5)]
    if flag == "rand":           # mixed signs, kept away from the poles of the divisions
        xs = [x * np.where(rs.rand(dim, dim) < 0.5, -1, 1).astype(np.float32) for x in xs]
    return xs


@pytest.mark.parametrize("f", [_compound_mix, _compound_transpose_mix], ids=["mix", "transpose_mix"])
@pytest.mark.parametrize("flag", ["pos_rand", "neg_rand", "rand"])
def test_compound_optree_oracle_vs_numpy(cpu, f, flag):
    xs = _compound_inputs(flag, 2)
    want = f(_Np(), *[x.astype(np.float64) for x in xs])
    out = cpu.empty((2, 2))
    out[:] = f(cpu, *[cpu.array(x) for x in xs])
    # the reference's own bar for these trees (rtol = atol = 1e-2)
    assert_close(out.get(), want.astype(np.float32), rtol=1e-2, atol=1e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("f", [_compound_mix, _compound_transpose_mix], ids=["mix", "transpose_mix"])
@pytest.mark.parametrize("flag", ["pos_rand", "neg_rand", "rand"])
@pytest.mark.parametrize("dim", [2, 40])
def test_compound_optree_hip(pair, f, flag, dim):
    xs = _compound_inputs(flag, dim)
    want = f(_Np(), *[x.astype(np.float64) for x in xs])
    got = []
    for be in pair:
        out = be.empty((dim, dim))
        out[:] = f(be, *[be.array(x) for x in xs])
        got.append(out.get())
    # chained products and reciprocals amplify rounding: compare both backends
    # with float64 at a tolerance scaled by the condition of the final division
    scale = max(1.0, np.abs(want).max())
    assert_close(got[0], want.astype(np.float32), rtol=1e-2, atol=1e-2 * scale)
    assert_close(got[1], want.astype(np.float32), rtol=1e-2, atol=1e-2 * scale)


# ---- batched_dot (reference tests/test_backend_batched_dot.py) -----------------------------------

def _batched_case(be, I, E, W, dtype):
    devI, devE, devW = (be.array(a.astype(dtype), dtype=dtype) for a in (I, E, W))
    devO, devB, devU = be.zeros(E.shape, dtype=dtype), be.zeros(I.shape, dtype=dtype), be.zeros(W.shape, dtype=dtype)
    be.batched_dot(devW, devI, devO)            # fprop
    be.batched_dot(devW.T, devE, devB)          # bprop
    be.batched_dot(devE, devI.T, devU)          # update
    return devO.get(), devB.get(), devU.get()


def _batched_data(X, N, C, K, seed=0):
    rs = np.random.RandomState(seed)
    return (rs.uniform(-1, 1, (X, C, N)), rs.uniform(-1, 1, (X, K, N)), rs.uniform(-1, 1, (K, C)))


def _batched_numpy(I, E, W):
    O = np.stack([W @ I[i] for i in range(I.shape[0])])
    B = np.stack([W.T @ E[i] for i in range(I.shape[0])])
    U = sum(E[i] @ I[i].T for i in range(I.shape[0]))
    return O, B, U


def test_batched_dot_oracle():
    from oracle import nervanacpu  # noqa: F401
    from neon_amd.backends.backend import Backend
    cpu = Backend.allocate_backend("cpu", rng_seed=0)
    I, E, W = _batched_data(5, 8, 24, 12)
    for got, want in zip(_batched_case(cpu, I, E, W, np.float32), _batched_numpy(I, E, W)):
        assert_close(got, want.astype(np.float32), rtol=0, atol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,atol", [(np.float32, 1e-3), (np.float16, 0.25)], ids=["f32", "f16"])
@pytest.mark.parametrize("X,N,C,K", [(100, 32, 1536, 768), (3, 5, 7, 9), (1, 64, 64, 64)])
def test_batched_dot_hip(hip, X, N, C, K, dtype, atol):
    I, E, W = _batched_data(X, N, C, K, seed=X)
    q = lambda a: a.astype(dtype).astype(np.float64)
    want = _batched_numpy(q(I), q(E), q(W))
    got = _batched_case(hip, I, E, W, dtype)
    for g, w in zip(got, want):
        # the reference's bar for fp32 (tests/test_backend_batched_dot.py: atol 1e-3); fp16 stores
        # sums of up to X*N = 3200 products
        assert_close(g.astype(np.float64), w, rtol=2e-3 if dtype == np.float16 else 0, atol=atol)


@pytest.mark.gpu
def test_batched_dot_alpha_beta_relu_hip(pair):
    I, E, W = _batched_data(4, 16, 40, 24, seed=2)
    res = []
    for be in pair:
        devI, devE, devW = (be.array(a.astype(np.float32)) for a in (I, E, W))
        O = be.array(E.astype(np.float32))
        U = be.array(W.astype(np.float32))
        be.batched_dot(devW, devI, O, alpha=0.5, beta=2.0)
        be.batched_dot(devE, devI.T, U, alpha=-1.5, beta=0.25)
        R = be.zeros(E.shape)
        be.batched_dot(devW, devI, R, relu=True)
        res.append((O.get(), U.get(), R.get()))
    for g, w in zip(res[1], res[0]):
        assert_close(g, w, rtol=1e-4, atol=1e-4)
    assert res[1][2].min() == 0.0
