"""
Activation functions (same names, arguments and formulas as the reference's
neon/transforms/activation.py).  Each call only *builds* an op-tree; the layer
that assigns it (``outputs[:] = act(inputs)``) triggers the fused kernel.
``bprop`` takes what the reference's takes: the function's output for
Tanh / Logistic, its input otherwise.
"""
from neon_amd.transforms.transform import Transform


class Identity(Transform):
    """f(x) = x"""

    def __call__(self, x):
        return x

    def bprop(self, x):
        return 1


class Rectlin(Transform):
    """max(x, 0) + slope * min(x, 0) (reference activation.py:56-95)"""

    def __init__(self, slope=0, name=None):
        super(Rectlin, self).__init__(name)
        self.slope = slope

    def __call__(self, x, nglayer=None):
        return self.be.fprop_relu(nglayer, x, self.slope)

    def bprop(self, x, nglayer=None, error=None, deltas=None):
        return self.be.bprop_relu(nglayer, x, error, deltas, self.slope)


class Rectlinclip(Transform):
    """leaky rectifier cut off at ``xcut`` (reference activation.py:98-114)"""

    def __init__(self, slope=0, name=None, xcut=20.0):
        super(Rectlinclip, self).__init__(name)
        self.xcut = xcut
        self.slope = slope

    def __call__(self, x):
        be = self.be
        return be.minimum(be.maximum(x, 0) + self.slope * be.minimum(x, 0), self.xcut)

    def bprop(self, x):
        be = self.be
        return (be.greater(x, 0) + self.slope * be.less(x, 0)) * be.greater(self.xcut, x)


class Explin(Transform):
    """max(x, 0) + alpha * (exp(min(x, 0)) - 1) (reference activation.py:117-156)"""

    def __init__(self, alpha=1.0, name=None):
        super(Explin, self).__init__(name)
        self.alpha = alpha

    def __call__(self, x):
        be = self.be
        return be.maximum(x, 0) + self.alpha * (be.exp(be.minimum(x, 0)) - 1)

    def bprop(self, x):
        # x is the function's output: for x <= 0 the derivative is x + alpha
        be = self.be
        return be.greater(x, 0) + be.minimum(x, 0) + self.alpha * be.less(x, 0)


class Normalizer(Transform):
    """x / divisor"""

    def __init__(self, name=None, divisor=128.):
        super(Normalizer, self).__init__(name)
        self.divisor = divisor

    def __call__(self, x):
        return x / self.divisor

    def bprop(self, x):
        return 1.0 / self.divisor


class Softmax(Transform):
    """exp(x - max) / sum(exp(x - max)) along ``axis``; the derivative is the
    shortcut 1, to be paired with a cross-entropy cost (reference
    activation.py:199-238)"""

    def __init__(self, axis=0, name=None, epsilon=2 ** -23):
        super(Softmax, self).__init__(name)
        self.epsilon = epsilon
        self.axis = axis

    def __call__(self, x):
        return self.be.fprop_softmax(x, self.axis)

    def bprop(self, x):
        return 1


class PixelwiseSoftmax(Transform):
    """Softmax over ``c`` channels for every pixel: the input (c * pixels,
    batch) is viewed as (c, pixels * batch) and normalised down each column, in
    place (reference activation.py:241-258)"""

    def __init__(self, c, name=None, epsilon=2 ** -23):
        super(PixelwiseSoftmax, self).__init__(name)
        self.epsilon = epsilon
        self.c = c

    def __call__(self, x):
        y = x.reshape((self.c, -1))
        shifted = self.be.exp(y - self.be.max(y, axis=0))
        y[:] = self.be.reciprocal(self.be.sum(shifted, axis=0)) * shifted
        return x

    def bprop(self, x):
        return 1


class Tanh(Transform):
    """tanh(x); derivative 1 - y^2 from the output y"""

    def __call__(self, x):
        return self.be.tanh(x)

    def bprop(self, x):
        return 1.0 - self.be.square(x)


class Logistic(Transform):
    """1 / (1 + exp(-x)); derivative y (1 - y) from the output y, or the
    shortcut 1 when paired with a cross-entropy cost (reference
    activation.py:296-360)"""

    def __init__(self, name=None, shortcut=False):
        super(Logistic, self).__init__(name)
        self.set_shortcut(shortcut)

    def set_shortcut(self, shortcut):
        self.shortcut = shortcut
        self.bprop_func = (lambda y: 1) if shortcut else (lambda y: y * (1.0 - y))

    def __call__(self, x):
        return self.be.sig(x)

    def bprop(self, y):
        return self.bprop_func(y)


class Sign(Transform):
    """+1 / -1 by the sign of x, in place (binary networks; reference
    activation.py:363-377); the straight-through derivative passes gradients
    where the stored input lies in [-1, 1]"""

    def __call__(self, x):
        return self.be.binarize(x, x, stochastic=False)

    def bprop(self, x):
        return self.be.less_equal(self.be.absolute(self.inputs), 1)
