"""
The sequential container (reference neon/layers/container.py: DeltasTree
:49-85, LayerContainer :88-180, Sequential :286-443): configures its layers in
order, lets the output-owning ones allocate, hands out two alternating shared
buffers for the back-propagated error and runs the passes.
"""
from neon_amd import NervanaObject
from neon_amd.layers.layer import Dropout, Layer


def _flatten(items):
    for item in items:
        if isinstance(item, (list, tuple)):
            for sub in _flatten(item):
                yield sub
        else:
            yield item


class DeltasTree(NervanaObject):
    """two buffers, each large enough for the largest layer input; consecutive
    delta-owning layers alternate between them"""

    def __init__(self):
        self.buffers = [None] * 2
        self.max_shape = 0

    def proc_layer(self, layer):
        in_size = layer.be.shared_iobuf_size(layer.in_shape, layer.parallelism)
        if in_size > self.max_shape:
            self.max_shape = in_size

    def allocate_buffers(self):
        for k in range(len(self.buffers)):
            if self.buffers[k] is None and self.max_shape > 0:
                self.buffers[k] = self.be.iobuf(self.max_shape, persist_values=False, parallelism="Data")


class Sequential(Layer):
    def __init__(self, layers, name=None):
        super(Sequential, self).__init__(name)
        self.layers = list(_flatten(layers))
        root = self.layers[0]
        assert root.owns_output or type(root) is Dropout, "Sequential root must own outputs"

    def __str__(self):
        return "\n".join(["Sequential '%s'" % self.name] + ["  " + str(layer) for layer in self.layers])

    @property
    def layers_to_optimize(self):
        lto = []
        for layer in self.layers:
            if isinstance(layer, Sequential):
                lto += layer.layers_to_optimize
            elif layer.has_params:
                if getattr(getattr(layer, "init", None), "name", None) == "Identity":
                    continue
                lto.append(layer)
        return lto

    def configure(self, in_obj):
        super(Sequential, self).configure(in_obj)
        prev = None
        for layer in self.layers:
            in_obj = layer.configure(in_obj)
            if prev is not None:
                prev.set_next(layer)
            prev = layer
        self.parallelism = in_obj.parallelism
        self.out_shape = in_obj.out_shape
        return self

    def allocate(self, shared_outputs=None):
        owners = [layer for layer in self.layers if layer.owns_output]
        owners[-1].allocate(shared_outputs)
        for layer in self.layers:
            layer.allocate()

    def allocate_deltas(self, global_deltas=None):
        if global_deltas is None:
            self.global_deltas = DeltasTree()
            for layer in self.layers[1:]:           # the first layer propagates to nobody
                layer.allocate_deltas(self.global_deltas)
            self.global_deltas.allocate_buffers()
        else:
            self.global_deltas = global_deltas
        self.set_deltas(self.global_deltas)

    def set_deltas(self, delta_buffers):
        for layer in self.layers:
            layer.set_deltas(delta_buffers)

    def fprop(self, inputs, inference=False, beta=0.0):
        x = inputs
        for layer in self.layers:
            if layer is self.layers[-1] and beta != 0:
                x = layer.fprop(x, inference=inference, beta=beta)
            else:
                x = layer.fprop(x, inference=inference)
        return x

    def bprop(self, error, alpha=1.0, beta=0.0):
        for layer in reversed(self.layers):
            if layer is self.layers[0]:
                error = layer.bprop(error, alpha, beta) if _takes_scale(layer) else layer.bprop(error)
            else:
                error = layer.bprop(error)
        return self.layers[0].deltas

    def get_terminal(self):
        return self.layers[-1].get_terminal()


def _takes_scale(layer):
    code = layer.bprop.__func__.__code__
    return "alpha" in code.co_varnames[:code.co_argcount]
