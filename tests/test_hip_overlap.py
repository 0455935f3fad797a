"""Statements whose output shares memory with one of their operands through
ANOTHER view.  The reference's CPU backend finishes the right-hand side before
it stores (nervanacpu.py:476-477: ``left[:] = right`` on a finished numpy
array); a kernel's lanes have no such order, so the hip backend has to notice
the overlap and evaluate through a temporary -- alone and inside fusion
groups.  Compared with the oracle element for element."""
import numpy as np
import pytest

from utils import assert_close, gen_inputs

pytestmark = pytest.mark.gpu


def _run(pair, program, shapes, seed, flag="rand"):
    rs = np.random.RandomState(seed)
    arrays = [gen_inputs(rs, s, flag) for s in shapes]
    outs = []
    for be in pair:
        tensors = [be.array(a) for a in arrays]
        program(be, *tensors)
        outs.append([t.get() for t in tensors])
    for got, want in zip(outs[1], outs[0]):
        assert_close(got, want)
    return outs


@pytest.mark.parametrize("shape", [(12, 8), (300, 257), (2000, 1024)])
def test_output_read_through_a_row_and_a_column_of_itself(pair, shape):
    def program(be, x, y):
        x[:] = y + x[2:3, :]                      # every row reads row 2, which the statement also writes
        x[:] = y * x[:, 1:2]                      # every column reads column 1
        x[:] = x - be.max(x, axis=0) + x[0:1, :]  # with a reduction of the output as well
    _run(pair, program, [shape, shape], 31)


@pytest.mark.parametrize("shape", [(12, 8), (513, 100)])
def test_reductions_of_a_tensor_written_into_slices_of_it(pair, shape):
    def program(be, x, y):
        x[:, 0:1] = be.sum(x, axis=1)
        x[0:1, :] = be.max(x, axis=0)
        x[:, 2:3] = be.sum(x * y, axis=1) + x[:, 3:4]
    _run(pair, program, [shape, shape], 32, "pos_rand")      # (positive terms: the sums' order does not show)


def test_shifted_copies_inside_one_tensor(pair):
    def program(be, x, y):
        x[1:] = x[:-1]                            # down by one row: numpy copies as if through a temporary
        x[:, :-3] = x[:, 3:] * 2.0                # left by three columns
        x[:-2] = x[2:] + y[2:]
    _run(pair, program, [(64, 40), (64, 40)], 33)


def test_fusion_groups_keep_statement_order_across_shifted_views(pair):
    """two statements that would each fuse, but the second reads, shifted by a
    row, what the first writes: one kernel would let the lane of row i read
    row i before the lane of row i-1 has written it"""
    from neon_amd.backends.backend import Block

    def in_a_minibatch_block(be, x, y, z):
        be.begin(Block.minibatch, 0)
        x[1:11] = y * 2.0
        z[:] = x[0:10] + 1.0
        z[:] = z + x[1:11]                        # the same view as the first statement wrote: may fuse
        x[0:10] = z * 0.5                         # writes over what the group wrote, shifted
        be.end(Block.minibatch, 0)
    _run(pair, in_a_minibatch_block, [(12, 8), (10, 8), (10, 8)], 34)

    def in_an_update_block(be, x, y, z):
        be.begin(Block.update, 0)
        x[2:12] = y * 3.0
        z[:] = x[1:11] - y
        be.end(Block.update, 0)
    _run(pair, in_an_update_block, [(12, 8), (10, 8), (10, 8)], 35)


def test_staging_happens_only_when_views_really_overlap(hip):
    x, y = hip.array(np.ones((16, 8), np.float32)), hip.array(np.ones((16, 8), np.float32))
    hip.synchronize()
    before = hip.plan_stats.get("staged", 0)
    x[:] = x * 2.0 + y                            # same elements
    x[0:8] = x[8:16] + 1.0                        # disjoint halves of one tensor
    x[:, 0:4] = x[:, 4:8] * y[:, 0:4]             # interleaved but disjoint columns (byte ranges do overlap)
    assert hip.plan_stats.get("staged", 0) - before <= 1
    x[:] = y + x[3:4, :]
    assert hip.plan_stats.get("staged", 0) - before >= 1
    want = np.ones((16, 8), np.float32) * 3.0
    want[0:8] = 4.0
    want[:, 0:4] = want[:, 4:8]
    want = 1.0 + want[3:4, :] + np.zeros_like(want)
    np.testing.assert_allclose(x.get(), want)
