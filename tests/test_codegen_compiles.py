"""Every shape class of the split column family is generated and compiled for
gfx950 with hiprtc (no GPU needed): trees with constants, fused outputs, pair
reductions, 16-bit storage, partial last column tiles, one chunk per strip."""
import numpy as np
import pytest

from neon_amd.backends import bfloat16
from neon_amd.backends.hip import prebuild


def _max(be, x, y):
    return [be.max(x, axis=0)]


def _argmax_and_max(be, x, y):
    return [be.argmax(x, axis=0), be.max(x, axis=0)]


def _argmin_of_expression(be, x, y):
    return [be.argmin(x * y - 0.25, axis=0)]


def _scaled_sum_of_products(be, x, y):
    return [be.sum(x * y * 2.5, axis=0) + 1.5]


def _sum_of_squares_about_a_number(be, x, y):
    return [be.sum(be.square(x - 0.5), axis=0)]


def _log_sum_exp(be, x, y):
    m = be.max(x, axis=0)
    return [be.log(be.sum(be.exp(x - m), axis=0)) + m]


TREES = [_max, _argmax_and_max, _argmin_of_expression, _scaled_sum_of_products,
         _sum_of_squares_about_a_number, _log_sum_exp]
SHAPES = [(32000, 256), (5000, 131), (70000, 32), (4096, 30000), (600, 7)]


@pytest.mark.parametrize("dtype", [np.float32, np.float16, bfloat16], ids=["f32", "f16", "bf16"])
@pytest.mark.parametrize("tree", TREES, ids=[t.__name__.strip("_") for t in TREES])
def test_split_column_kernels_compile(tmp_path, tree, dtype):
    be = prebuild.PlanBackend(cache_dir=str(tmp_path / "kc"), compile_kernels=True)
    families = set()
    for shape in SHAPES:
        x, y = be.empty(shape, dtype), be.empty(shape, dtype)
        exprs = tree(be, x, y)
        outs = [be.empty((1, shape[1]), np.int32 if "arg" in e[0]["op"] else np.float32) for e in exprs]
        be.begin(prebuild.Block.update, 0)
        for o, e in zip(outs, exprs):
            o[:] = e
        be.end(prebuild.Block.update, 0)
        families.add(be.choices[-1].spec.family)
    assert "colsplit" in families
