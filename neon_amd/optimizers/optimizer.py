"""
Learning-rate schedules and parameter update rules (the role of
neon/optimizers/optimizer.py in the reference; same class names, constructor
arguments and update formulas).

Every rule is written against the backend's tensor API only: a handful of
``tensor[:] = expr`` statements per parameter.  Each parameter's statements are
bracketed by ``be.begin(Block.update, i)`` / ``be.end(Block.update, i)`` -- hooks
the reference declares as optimisation hints (backend.py:671-709) -- which lets
the hip backend run them as ONE kernel that reads and writes every tensor once
(Adam: 4 reads + 3 writes instead of 10 passes).  Backends that ignore the
hooks execute the same statements one by one with the same results.

A layer is anything with ``get_params()`` returning ``((W, dW), states)`` or a
list of such tuples, ``states`` being a list the optimizer fills on first use
(reference optimizer.py:25-41).
"""
import numpy as np

from neon_amd import NervanaObject
from neon_amd.backends.backend import Block


def get_param_list(layer_list):
    """flat list of ``((W, dW), states)`` over all layers"""
    params = []
    for layer in layer_list:
        got = layer.get_params()
        if isinstance(got, list):
            params.extend(got)
        else:
            params.append(got)
    return params


# ---------------------------------------------------------------------------------------
# schedules (reference optimizer.py:118-414)
# ---------------------------------------------------------------------------------------
class Schedule(NervanaObject):
    """Constant rate, or ``rate * change ** steps`` with ``steps`` the number of
    entries of ``step_config`` (a list of epochs) already passed -- or
    ``epoch // step_config`` for an integer ``step_config``.  With two lists the
    rate is *set* to ``change[i]`` from epoch ``step_config[i]`` on."""

    def __init__(self, step_config=None, change=1.):
        if isinstance(step_config, list) and isinstance(change, list):
            assert len(step_config) == len(change), "change and step_config must have the same length"
        self.step_config = step_config
        self.change = change
        self.steps = 0

    def get_learning_rate(self, learning_rate, epoch):
        if isinstance(self.step_config, list) and isinstance(self.change, list):
            if epoch in self.step_config:
                self.steps = self.change[self.step_config.index(epoch)]
            return learning_rate if self.steps == 0 else self.steps
        if isinstance(self.step_config, int):
            self.steps = np.floor(epoch / self.step_config)
        elif isinstance(self.step_config, list):
            self.steps = np.sum(epoch >= np.array(self.step_config))
        return float(learning_rate * self.change ** self.steps)


class StepSchedule(Schedule):
    """rate set to ``change[i]`` from epoch ``step_config[i]`` on"""

    def __init__(self, step_config, change):
        assert isinstance(step_config, list) and isinstance(change, list), \
            "The arguments change and step_config must be lists."
        assert len(step_config) == len(change), \
            "The arguments change and step_config must have the same length."
        self.step_config, self.change, self.steps = step_config, change, 0

    def get_learning_rate(self, learning_rate, epoch):
        if epoch in self.step_config:
            self.steps = self.change[self.step_config.index(epoch)]      # holds the current rate
        return learning_rate if self.steps == 0 else self.steps


class PowerSchedule(Schedule):
    """``rate * change ** (epoch // step_config)``"""

    def __init__(self, step_config, change):
        assert isinstance(step_config, int), "The argument step_config must be an integer."
        assert not isinstance(change, list), "The argument change must be a float or integer."
        self.step_config, self.change, self.steps = step_config, change, 0

    def get_learning_rate(self, learning_rate, epoch):
        self.steps = np.floor(epoch / self.step_config)
        return float(learning_rate * self.change ** self.steps)


class ExpSchedule(Schedule):
    """``rate / (1 + decay * epoch)``"""

    def __init__(self, decay):
        self.decay = decay

    def get_learning_rate(self, learning_rate, epoch):
        return float(learning_rate / (1. + self.decay * epoch))


class PolySchedule(Schedule):
    """``rate * (1 - epoch // total_epochs) ** power``"""

    def __init__(self, total_epochs, power):
        self.total_epochs = np.float32(total_epochs)
        self.power = power

    def get_learning_rate(self, learning_rate, epoch):
        return float(learning_rate * (1. - epoch // self.total_epochs) ** self.power)


class ShiftSchedule(Schedule):
    """rate halved (``shift_size`` binary places) every ``interval`` epochs"""

    def __init__(self, interval, shift_size=1):
        self.interval = interval
        self.shift_size = shift_size

    def get_learning_rate(self, learning_rate, epoch):
        total_shift = -1 * self.shift_size * int(epoch / self.interval)
        return float(self.be.shift(learning_rate, total_shift, value=False).get().reshape(-1)[0])


# ---------------------------------------------------------------------------------------
# update rules
# ---------------------------------------------------------------------------------------
class Optimizer(NervanaObject):
    """Base: gradient-norm scaling, value clipping and the per-parameter loop."""

    def __init__(self, name=None):
        self.name = name or self.__class__.__name__

    def optimize(self, layer_list, epoch):
        raise NotImplementedError()

    def clip_gradient_norm(self, param_list, clip_norm):
        """factor (<= 1) that brings the gradients' global L2 norm, divided by
        the batch size, down to ``clip_norm`` (reference optimizer.py:72-96)"""
        if not clip_norm:
            return 1
        be = self.be
        total = sum(be.sum(be.square(grad)) for (param, grad), states in param_list)
        norm = be.zeros((1, 1))
        norm[:] = be.sqrt(total) / be.bsz
        return clip_norm / max(float(norm.get().reshape(-1)[0]), float(clip_norm))

    def clip_value(self, v, abs_bound=None):
        if abs_bound:
            return self.be.clip(v, -abs(abs_bound), abs(abs_bound))
        return v

    def _updates(self, layer_list, n_states):
        """yield (param, grad / batch size, states) per parameter, with the
        states created on first use and the statements the caller issues in
        between fused into one update group"""
        be = self.be
        for i, ((param, grad), states) in enumerate(get_param_list(layer_list)):
            param.rounding = self.stochastic_round
            if len(states) == 0:
                states.extend(be.zeros_like(grad) for _ in range(n_states))
            be.begin(Block.update, i)
            try:
                yield param, grad / be.bsz, states
            finally:
                be.end(Block.update, i)


class GradientDescentMomentum(Optimizer):
    """``v = mu * v - lr * (s * g + wd * W);  W += v`` (or the Nesterov form
    ``W += mu * v - lr * g'``); without momentum ``W = -lr * s * g + (1 - lr * wd) * W``
    (reference optimizer.py:416-540)."""

    def __init__(self, learning_rate, momentum_coef, stochastic_round=False, wdecay=0.0,
                 gradient_clip_norm=None, gradient_clip_value=None, param_clip_value=None,
                 name=None, schedule=None, nesterov=False):
        super(GradientDescentMomentum, self).__init__(name=name)
        self.learning_rate, self.momentum_coef = learning_rate, momentum_coef
        self.gradient_clip_norm = gradient_clip_norm
        self.gradient_clip_value = gradient_clip_value
        self.param_clip_value = param_clip_value
        self.wdecay = wdecay
        self.schedule = schedule if schedule is not None else Schedule()
        self.stochastic_round = stochastic_round
        self.nesterov = nesterov
        if self.momentum_coef == 0 and self.nesterov:
            raise ValueError("nesterov requires non-zero momentum")

    def optimize(self, layer_list, epoch):
        lrate = self.schedule.get_learning_rate(self.learning_rate, epoch)
        scale = self.clip_gradient_norm(get_param_list(layer_list), self.gradient_clip_norm)
        mu = self.momentum_coef
        for param, grad, states in self._updates(layer_list, 1 if mu != 0 else 0):
            grad = self.clip_value(grad, self.gradient_clip_value)
            if mu == 0:
                # (the reference builds a clipped tree here but never assigns it,
                # optimizer.py:519-521: without momentum the parameters are not clipped)
                param[:] = (-lrate * scale) * grad + (1 - lrate * self.wdecay) * param
                continue
            grad = scale * grad + self.wdecay * param
            velocity = states[0]
            velocity[:] = mu * velocity - lrate * grad
            if self.nesterov:
                param[:] = self.clip_value(param + mu * velocity - lrate * grad, self.param_clip_value)
            else:
                param[:] = self.clip_value(param + velocity, self.param_clip_value)


class RMSProp(Optimizer):
    """``r = d * r + (1 - d) * g^2;  W -= s * g * lr / (sqrt(r + eps) + eps)``
    (reference optimizer.py:542-634)."""

    def __init__(self, stochastic_round=False, decay_rate=0.95, learning_rate=2e-3, epsilon=1e-6,
                 gradient_clip_norm=None, gradient_clip_value=None, param_clip_value=None,
                 name=None, schedule=None):
        super(RMSProp, self).__init__(name=name)
        self.epsilon, self.decay_rate, self.learning_rate = epsilon, decay_rate, learning_rate
        self.schedule = schedule if schedule is not None else Schedule()
        self.gradient_clip_norm = gradient_clip_norm
        self.gradient_clip_value = gradient_clip_value
        self.param_clip_value = param_clip_value
        self.stochastic_round = stochastic_round

    def optimize(self, layer_list, epoch):
        be = self.be
        lrate = self.schedule.get_learning_rate(self.learning_rate, epoch)
        eps, decay = self.epsilon, self.decay_rate
        scale = self.clip_gradient_norm(get_param_list(layer_list), self.gradient_clip_norm)
        for param, grad, (state,) in self._updates(layer_list, 1):
            grad = self.clip_value(grad, self.gradient_clip_value)
            state[:] = decay * state + be.square(grad) * (1.0 - decay)
            param[:] = self.clip_value(param - (scale * grad * lrate) / (be.sqrt(state + eps) + eps),
                                       self.param_clip_value)


class Adagrad(Optimizer):
    """``h += g^2;  W -= s * g * lr / sqrt(h + eps)`` (reference optimizer.py:636-731)."""

    def __init__(self, stochastic_round=False, learning_rate=0.01, epsilon=1e-6,
                 gradient_clip_norm=None, gradient_clip_value=None, param_clip_value=None, name=None):
        super(Adagrad, self).__init__(name=name)
        self.epsilon, self.learning_rate = epsilon, learning_rate
        self.gradient_clip_norm = gradient_clip_norm
        self.gradient_clip_value = gradient_clip_value
        self.param_clip_value = param_clip_value
        self.stochastic_round = stochastic_round

    def optimize(self, layer_list, epoch):
        be = self.be
        lrate, eps = self.learning_rate, self.epsilon
        scale = self.clip_gradient_norm(get_param_list(layer_list), self.gradient_clip_norm)
        for param, grad, (state,) in self._updates(layer_list, 1):
            grad = self.clip_value(grad, self.gradient_clip_value)
            state[:] = state + be.square(grad)
            param[:] = self.clip_value(param - (scale * grad * lrate) / be.sqrt(state + eps),
                                       self.param_clip_value)


class Adadelta(Optimizer):
    """``E[g^2] = d E[g^2] + (1-d) g^2;  u = sqrt((E[u^2] + eps) / (E[g^2] + eps)) g;
    E[u^2] = d E[u^2] + (1-d) u^2;  W -= u`` (reference optimizer.py:733-823)."""

    def __init__(self, stochastic_round=False, decay=0.95, epsilon=1e-6, param_clip_value=None, name=None):
        super(Adadelta, self).__init__(name=name)
        self.decay, self.epsilon = decay, epsilon
        self.stochastic_round = stochastic_round
        self.param_clip_value = param_clip_value

    def optimize(self, layer_list, epoch):
        be = self.be
        eps, decay = self.epsilon, self.decay
        for param, grad, (gsq, usq, upd) in self._updates(layer_list, 3):
            gsq[:] = gsq * decay + (1. - decay) * grad * grad
            upd[:] = be.sqrt((usq + eps) / (gsq + eps)) * grad
            usq[:] = usq * decay + (1. - decay) * upd * upd
            param[:] = self.clip_value(param - upd, self.param_clip_value)


class Adam(Optimizer):
    """``m = b1 m + (1-b1) g;  v = b2 v + (1-b2) g^2;
    W -= s * lr * sqrt(1 - b2^t) / (1 - b1^t) * m / (sqrt(v) + eps)``
    (reference optimizer.py:825-930)."""

    def __init__(self, stochastic_round=False, learning_rate=0.001, beta_1=0.9, beta_2=0.999,
                 epsilon=1e-8, gradient_clip_norm=None, gradient_clip_value=None,
                 param_clip_value=None, name="adam"):
        super(Adam, self).__init__(name=name)
        self.beta_1, self.beta_2, self.epsilon = beta_1, beta_2, epsilon
        self.learning_rate = learning_rate
        self.stochastic_round = stochastic_round
        self.gradient_clip_norm = gradient_clip_norm
        self.gradient_clip_value = gradient_clip_value
        self.param_clip_value = param_clip_value
        self.t = 0

    def optimize(self, layer_list, epoch):
        be = self.be
        self.t = self.t + 1
        step = self.learning_rate * be.sqrt(1 - self.beta_2 ** self.t) / (1 - self.beta_1 ** self.t)
        scale = self.clip_gradient_norm(get_param_list(layer_list), self.gradient_clip_norm)
        for param, grad, (m, v) in self._updates(layer_list, 2):
            grad = self.clip_value(grad, self.gradient_clip_value)
            m[:] = m * self.beta_1 + (1. - self.beta_1) * grad
            v[:] = v * self.beta_2 + (1. - self.beta_2) * grad * grad
            param[:] = self.clip_value(param - (scale * step * m) / (be.sqrt(v) + self.epsilon),
                                       self.param_clip_value)


class ShiftAdaMax(Optimizer):
    """AdaMax whose scalings are rounded to powers of two (binary networks):
    ``m = b1 m + (1-b1) g;  v = max(b2 v, |g|);  W -= shift(shift(m, 1/(v+eps)), lr / (1 - b1^t))``,
    ``W`` kept in [-1, 1] (reference optimizer.py:933-990)."""

    def __init__(self, stochastic_round=False, learning_rate=0.002, beta_1=0.9, beta_2=0.999,
                 epsilon=1e-8, schedule=None, name="ShiftAdaMax"):
        super(ShiftAdaMax, self).__init__(name=name)
        self.beta_1, self.beta_2, self.epsilon = beta_1, beta_2, epsilon
        self.learning_rate = learning_rate
        self.stochastic_round = stochastic_round
        self.schedule = schedule if schedule is not None else Schedule()

    def optimize(self, layer_list, epoch):
        be = self.be
        t = epoch + 1
        lrate = self.schedule.get_learning_rate(self.learning_rate, epoch)
        step = lrate / (1 - self.beta_1 ** t)
        for (param, grad), states in get_param_list(layer_list):
            param.rounding = self.stochastic_round
            if len(states) == 0:
                states.extend(be.zeros_like(grad) for _ in range(3))
            grad = grad / be.bsz
            m, v, inv_v = states
            m[:] = m * self.beta_1 + (1. - self.beta_1) * grad
            v[:] = be.maximum(v * self.beta_2, be.absolute(grad))
            inv_v[:] = 1.0 / (v + self.epsilon)
            param[:] = param - be.shift(be.shift(m, inv_v), step)
            be.clip(param, -1, 1, param)


class MultiOptimizer(Optimizer):
    """Different rules for different layers: ``optimizer_mapping`` maps a layer's
    ``name`` or class name to an optimizer, ``'default'`` catches the rest
    (reference optimizer.py:993-1138)."""

    def __init__(self, optimizer_mapping, name=None):
        super(MultiOptimizer, self).__init__(name=name)
        assert "default" in optimizer_mapping, "Must specify a default optimizer in layer type to optimizer mapping"
        self.optimizer_mapping = optimizer_mapping
        self.map_list = None

    def _map_optimizers(self, layer_list):
        groups = {}
        for layer in layer_list:
            cls, name = layer.__class__.__name__, getattr(layer, "name", None)
            if name in self.optimizer_mapping:
                opt = self.optimizer_mapping[name]
            elif cls in self.optimizer_mapping:
                opt = self.optimizer_mapping[cls]
            else:
                opt = self.optimizer_mapping["default"]
            groups.setdefault(opt, []).append(layer)
        return groups

    def optimize(self, layer_list, epoch):
        if self.map_list is None:
            self.map_list = self._map_optimizers(layer_list)
        for opt, layers in self.map_list.items():
            opt.optimize(layers, epoch)
