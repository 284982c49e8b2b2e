"""The four neon formulas that define the fused benchmark graphs.

Only the op sequences are taken over from the reference front end, so the
graphs the backend fuses are the ones the reference would hand it:

* `batch_norm_train`  ngraph/frontends/neon/layer.py:1242-1257
* `adam_update`       ngraph/frontends/neon/optimizer.py:446-470
* `lstm_cell`         ngraph/frontends/neon/layer.py:1630-1647 (gate order i,f,o,g :1615)
* `rectlin`           ngraph/frontends/neon/activation.py:46

plus the other elementwise pieces a training step is made of on this path: the activation
classes, Dropout, two cost formulas and the learning rules.
"""
import numpy as np

import ngraph_hip as ng


def rectlin(x, slope=0):
    return ng.maximum(x, 0) + slope * ng.minimum(0, x)


# ---- activations (ngraph/frontends/neon/activation.py:21-190): elementwise composites that
# ---- the backend fuses into their producer ---------------------------------------------------
class Rectlin(object):
    def __init__(self, slope=0, **kwargs):
        self.slope = slope

    def __call__(self, x):
        return ng.maximum(x, 0) + self.slope * ng.minimum(0, x)


class Rectlinclip(object):
    def __init__(self, slope=0, cutoff=20.0, name=None):
        self.cutoff, self.slope = cutoff, slope

    def __call__(self, x):
        return ng.minimum(ng.maximum(x, 0) + self.slope * ng.minimum(x, 0), self.cutoff)


class Identity(object):
    def __call__(self, x):
        return x


class Explin(object):
    def __init__(self, alpha=1.0):
        self.alpha = alpha

    def __call__(self, x):
        return ng.maximum(x, 0) + self.alpha * (ng.exp(ng.minimum(x, 0)) - 1)


class Normalizer(object):
    def __init__(self, divisor=128.):
        self.divisor = divisor

    def __call__(self, x):
        return x / self.divisor


class Softmax(object):
    def __call__(self, x):
        return ng.softmax(x)


class Tanh(object):
    def __call__(self, x):
        return ng.tanh(x)


class Logistic(object):
    def __call__(self, x):
        return ng.sigmoid(x)


class Dropout(object):
    """Training: a fresh uniform mask per execution, `(u <= keep) * x`; inference: `keep * x`
    (ngraph/frontends/neon/layer.py:1272-1303).  The random fill is an op of the fused kernel,
    so mask and product are one launch."""

    inference_mode = False

    def __init__(self, keep=0.5, **kwargs):
        self.keep = keep
        self.mask = None

    def __call__(self, in_obj):
        if Dropout.inference_mode:
            return self.keep * in_obj
        if self.mask is None:
            self.mask = ng.persistent_tensor(axes=in_obj.axes.sample_axes())
        self.mask = ng.uniform(self.mask, low=0.0, high=1.0) <= self.keep
        return self.mask * in_obj


# ---- costs as the reference's tests build them (neon/tests/test_costs.py:46-76) ---------------
def sum_squared(y, t):
    return ng.squared_L2(y - t, out_axes=()) / 2


def mean_squared(y, t):
    return ng.mean(ng.square(y - t), out_axes=()) / 2.


def batch_norm_train(in_obj, gamma, beta, out_axes, eps=1e-5):
    """Training-mode normalisation of `in_obj` over every axis not in out_axes.

    Returns (y, xmean, xvar); the caller may also assign running statistics.
    """
    out_axes = ng.make_axes(out_axes)
    red_axes = in_obj.axes - out_axes
    flat = ng.flatten(ng.axes_with_order(in_obj, out_axes | red_axes),
                      out_axes | red_axes.flatten(force=True))
    xmean = ng.mean(flat, out_axes=out_axes)
    xvar = ng.variance(flat, out_axes=out_axes)
    y = ng.unflatten(gamma * ((flat - xmean) * ng.reciprocal(ng.sqrt(xvar + eps))) + beta)
    return y, xmean, xvar


class Adam(object):
    """Adam learning rule; `__call__` advances t, `variable_update` builds one update."""

    def __init__(self, learning_rate=1e-3, beta_1=0.9, beta_2=0.999, epsilon=1e-8):
        self.lrate = learning_rate
        self.beta_1 = ng.constant(beta_1, dtype=np.float32)
        self.beta_2 = ng.constant(beta_2, dtype=np.float32)
        self.epsilon = epsilon
        self.t = ng.persistent_tensor(axes=(), initial_value=0)
        self.step = None
        self.ell = None

    def __call__(self):
        self.step = ng.sequential([ng.assign(self.t, self.t + 1), self.t])
        self.ell = self.lrate * ng.sqrt(1 - self.beta_2 ** self.step) / (1 - self.beta_1 ** self.step)
        return self.ell

    def variable_update(self, variable, grad, scale_factor=1):
        m = ng.persistent_tensor(axes=grad.axes, initial_value=0.)
        v = ng.persistent_tensor(axes=grad.axes, initial_value=0.)
        updates = ng.sequential([
            ng.assign(m, m * self.beta_1 + (1 - self.beta_1) * grad),
            ng.assign(v, v * self.beta_2 + (1 - self.beta_2) * grad * grad),
            ng.assign(variable,
                      variable - (scale_factor * self.ell * m) / (ng.sqrt(v) + self.epsilon))
        ])
        return updates, m, v


class GradientDescentMomentum(object):
    """SGD with momentum, weight decay, optional Nesterov step and the Kahan-compensated
    parameter update of frontends/neon/optimizer.py:285-310."""

    def __init__(self, learning_rate, momentum_coef=0.0, wdecay=0.0, nesterov=False):
        self.lrate = learning_rate
        self.momentum_coef = momentum_coef
        self.wdecay = wdecay
        self.nesterov = nesterov

    def variable_update(self, variable, grad, scale_factor=1):
        velocity = ng.persistent_tensor(axes=variable.axes, initial_value=0.)
        lr = - self.lrate * (scale_factor * grad + self.wdecay * variable)
        updates = [ng.assign(velocity, velocity * self.momentum_coef + lr)]
        delta = (self.momentum_coef * velocity + lr) if self.nesterov else velocity
        kahan_c = ng.persistent_tensor(axes=variable.axes, initial_value=0.)
        kahan_y = ng.persistent_tensor(axes=variable.axes, initial_value=0.)
        kahan_t = ng.persistent_tensor(axes=variable.axes, initial_value=0.)
        updates.append(ng.assign(kahan_y, delta - kahan_c))
        updates.append(ng.assign(kahan_t, variable + kahan_y))
        updates.append(ng.assign(kahan_c, (kahan_t - variable) - kahan_y))
        updates.append(ng.assign(variable, kahan_t))
        return ng.sequential(updates), velocity


class RMSProp(object):
    """frontends/neon/optimizer.py:370-383."""

    def __init__(self, decay_rate=0.95, learning_rate=2e-3, epsilon=1e-6, wdecay=0.0, momentum_coef=0.0):
        self.decay_rate, self.lrate, self.epsilon = decay_rate, learning_rate, epsilon
        self.wdecay, self.momentum = wdecay, momentum_coef

    def variable_update(self, variable, grad, scale_factor=1):
        epsilon, decay = self.epsilon, self.decay_rate
        state = ng.persistent_tensor(axes=variable.axes, initial_value=1.)
        velocity = ng.persistent_tensor(axes=variable.axes, initial_value=0.)
        updates = ng.sequential([
            ng.assign(state, decay * state + (1.0 - decay) * ng.square(grad)),
            ng.assign(velocity, velocity * self.momentum +
                      (self.lrate * scale_factor * grad / ng.sqrt(state + epsilon)) +
                      self.lrate * self.wdecay * variable),
            ng.assign(variable, variable - velocity)
        ])
        return updates, state, velocity


class Adagrad(object):
    """frontends/neon/optimizer.py:533-542."""

    def __init__(self, learning_rate=0.01, epsilon=1e-6):
        self.lrate, self.epsilon = learning_rate, epsilon

    def variable_update(self, variable, grad, scale_factor=1):
        state = ng.persistent_tensor(axes=grad.axes, initial_value=0.)
        updates = ng.sequential([
            ng.assign(state, state + ng.square(grad)),
            ng.assign(variable,
                      variable - (scale_factor * self.lrate * grad) / (ng.sqrt(state + self.epsilon)))
        ])
        return updates, state


def lstm_cell(gates, c_prev, hidden_axis, gate_slices):
    """Pointwise part of an LSTM step.

    gates: dict k -> pre-activation [H, N] for k in i, f, o, g.
    Returns (h, c).
    """
    act = {k: ng.tanh(gates[k]) if k == "g" else ng.sigmoid(gates[k]) for k in ("i", "f", "o", "g")}
    c = act["f"] * c_prev + act["i"] * act["g"]
    h = act["o"] * ng.tanh(c)
    return h, c
