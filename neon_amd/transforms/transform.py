"""Base of activation and cost functions (reference neon/transforms/transform.py)."""
from neon_amd import NervanaObject


class Transform(NervanaObject):
    """``__call__`` gives f(x) and ``bprop`` its derivative, both as op-trees;
    subclasses override them or set ``self.func`` / ``self.funcgrad``."""

    def __init__(self, name=None):
        self.name = name or self.__class__.__name__

    def __call__(self, x):
        return self.func(x)

    def bprop(self, x):
        return self.funcgrad(x)
