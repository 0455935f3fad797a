"""
Reverse-mode differentiation of op-trees.

A pure client of the tensor API (the role of neon/backends/autodiff.py in the
reference): given an op-tree ``f`` it produces, for every tensor in it, another
op-tree for d(sum(f * next_error))/d(tensor).  Nothing is computed until a
gradient tree is assigned, at which point it runs through ``backend.execute``
like any other tree -- on the hip backend as fused kernels, reductions that
undo broadcasts included.

Public surface as in the reference (autodiff.py:338-480): ``Autodiff(op_tree,
be, next_error=None)`` with ``back_prop_grad``, ``get_grad_op_tree``,
``get_grad_tensor``, ``get_grad_asnumpyarray`` and ``cleanup``.

How it works: one walk from the root down.  Each node turns the gradient that
arrives for its value into gradients for its operands with a local rule
(``_RULES``), shrinks them back to the operands' shapes where the forward op
broadcast (``_unbroadcast``), and passes them on; gradients reaching the same
tensor from several paths add up.
"""
import numpy as np

from neon_amd.backends.backend import OpTreeNode, Tensor

_NUMBER = (int, float)
_LN2 = float(np.log(2.0))


def _shape_of(x):
    if isinstance(x, (Tensor, OpTreeNode)):
        shape = tuple(x.shape)
        return shape + (1,) if len(shape) == 1 else shape
    return (1, 1)


def _unbroadcast(grad, operand, be):
    """Gradient for ``operand`` from a gradient of the op's (possibly larger or
    smaller) result shape.  Broadcast forward => sum backward; a reduction
    forward => spread the gradient back over the reduced axis."""
    if grad is None or operand is None:
        return None
    if isinstance(operand, _NUMBER):
        return None
    want, have = _shape_of(operand), _shape_of(grad)
    if want == have:
        return grad
    if len(want) != 2 or len(have) != 2:
        raise NotImplementedError("gradients of broadcasts beyond two dimensions")
    if want == (1, 1):
        return be.sum(grad)                       # 1x1 operand fed every element
    if want[0] == have[0] and want[1] == 1:
        return be.sum(grad, axis=1)               # column vector broadcast along rows
    if want[0] == 1 and want[1] == have[1]:
        return be.sum(grad, axis=0)               # row vector broadcast down columns
    if (have[0] == want[0] and have[1] == 1) or (have[0] == 1 and have[1] == want[1]) or have == (1, 1):
        return 0 * operand + grad                 # forward op reduced: every element gets the gradient
    raise NotImplementedError("cannot map a gradient of shape %s onto an operand of shape %s" % (have, want))


# local rules: (x, y, z, dz, be) -> (dL/dx, dL/dy); z is the node's own value
_RULES = {
    "add": lambda x, y, z, dz, be: (dz, dz),
    "sub": lambda x, y, z, dz, be: (dz, -dz),
    "mul": lambda x, y, z, dz, be: (dz * y, dz * x),
    "div": lambda x, y, z, dz, be: (dz / y, -dz * x / be.square(y)),
    "pow": lambda x, y, z, dz, be: (dz * y * x ** (y - 1.), dz * z * be.log(x)),
    "neg": lambda x, y, z, dz, be: (-dz, None),
    "abs": lambda x, y, z, dz, be: (dz * be.sgn(x), None),
    "sqrt": lambda x, y, z, dz, be: (dz * 0.5 / z, None),
    "sqr": lambda x, y, z, dz, be: (dz * 2. * x, None),
    "exp": lambda x, y, z, dz, be: (dz * z, None),
    "exp2": lambda x, y, z, dz, be: (dz * z * _LN2, None),
    "log": lambda x, y, z, dz, be: (dz / x, None),
    "safelog": lambda x, y, z, dz, be: (dz / x, None),
    "log2": lambda x, y, z, dz, be: (dz / x / _LN2, None),
    "sig": lambda x, y, z, dz, be: (dz * z * (1. - z), None),
    "sig2": lambda x, y, z, dz, be: (dz * z * (1. - z) * _LN2, None),
    "tanh": lambda x, y, z, dz, be: (dz * (1. - be.square(z)), None),
    "tanh2": lambda x, y, z, dz, be: (dz * (1. - be.square(z)) * _LN2, None),
    "maximum": lambda x, y, z, dz, be: (dz * be.greater_equal(x, y), dz * be.greater_equal(y, x)),
    "minimum": lambda x, y, z, dz, be: (dz * be.less_equal(x, y), dz * be.less_equal(y, x)),
    # reductions: the gradient is spread back by _unbroadcast; max/min only
    # reach the elements that attained the extreme
    "sum": lambda x, y, z, dz, be: (dz, None),
    "max": lambda x, y, z, dz, be: (dz * be.equal(x, z), None),
    "min": lambda x, y, z, dz, be: (dz * be.equal(x, z), None),
    "transpose": lambda x, y, z, dz, be: (dz.T, None),
    "dot": lambda x, y, z, dz, be: (be.dot(dz, y.T), be.dot(x.T, dz)),
}
# piecewise-constant ops: no gradient flows through them
_FLAT = {"eq", "ne", "lt", "le", "gt", "ge", "sgn", "finite", "argmax", "argmin", "rint", "onehot", "rand"}


class Autodiff(object):
    """Gradient op-trees of ``op_tree`` with respect to the tensors in it.

    ``next_error`` (same shape as ``op_tree``) is the gradient arriving from
    whatever consumes the tree's value; ones by default."""

    def __init__(self, op_tree, be, next_error=None):
        assert isinstance(op_tree, _NUMBER + (OpTreeNode, Tensor)), "op_tree type not supported"
        assert be is not None
        self.op_tree = op_tree
        self.be = be
        self.dtype = be.default_dtype
        if next_error is not None:
            assert tuple(next_error.shape) == _shape_of(op_tree), (
                "next_error.shape %s must be consistant with op_tree.shape %s"
                % (next_error.shape, _shape_of(op_tree)))
            self.next_error = next_error
        else:
            self.next_error = be.ones(_shape_of(op_tree))
        self.map_tensor_grad_op_tree = {}
        self._descend(op_tree, self.next_error)

    # -- the walk ------------------------------------------------------------------------
    def _descend(self, node, dz):
        if dz is None or node is None or isinstance(node, _NUMBER):
            return
        if isinstance(node, Tensor):
            key = node.get_original_base()
            have = self.map_tensor_grad_op_tree.get(key)
            self.map_tensor_grad_op_tree[key] = dz if have is None else have + dz
            return
        op = node[0]["op"]
        if op in _FLAT:
            return
        rule = _RULES.get(op)
        if rule is None:
            raise NotImplementedError("no derivative rule for op '%s'" % op)
        x, y = node[1], node[2]
        if op in ("sum", "max", "min") and node[0].get("axis") not in (0, 1):
            raise NotImplementedError("gradient of a reduction without an axis")
        gx, gy = rule(x, y, node, dz, self.be)
        self._descend(x, _unbroadcast(gx, x, self.be))
        self._descend(y, _unbroadcast(gy, y, self.be))

    # -- results (reference autodiff.py:414-480) ----------------------------------------------
    def get_grad_op_tree(self, tensors):
        """gradient op-tree for each tensor (a zero tree for tensors ``op_tree``
        does not depend on)"""
        return [self.map_tensor_grad_op_tree.get(t.get_original_base(), t * 0.) for t in tensors]

    def get_grad_tensor(self, tensors):
        out = []
        for tree in self.get_grad_op_tree(tensors):
            buf = self.be.empty(_shape_of(tree))
            buf[:] = tree
            out.append(buf)
        return out

    def get_grad_asnumpyarray(self, tensors):
        return [t.get().astype(self.dtype) for t in self.get_grad_tensor(tensors)]

    def back_prop_grad(self, tensors, gradients):
        """evaluate the gradients of ``tensors`` into the buffers ``gradients``;
        ``next_error`` may itself be one of the buffers (it is written last)"""
        for buf in gradients:
            assert buf.get_original_base() not in self.map_tensor_grad_op_tree, \
                "a tensor of the tree cannot also receive a gradient"
        deferred = None
        for t, buf in zip(tensors, gradients):
            if buf is self.next_error:
                deferred = t
            else:
                buf[:] = self.map_tensor_grad_op_tree.get(t.get_original_base(), buf * 0.)
        if deferred is not None:
            self.next_error[:] = self.map_tensor_grad_op_tree.get(deferred.get_original_base(),
                                                                  self.next_error * 0.)

    def cleanup(self):
        self.map_tensor_grad_op_tree = {}
        self.next_error = None
        self.op_tree = None
        self.be = None
