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
    rstd = ng.reciprocal(ng.sqrt(xvar + eps))
    y = ng.unflatten(gamma * ((flat - xmean) * rstd) + beta)
    y.deriv_handler = _BatchNormAdjoint(flat, gamma, beta, xmean, rstd, out_axes)
    return y, xmean, xvar


class _BatchNormAdjoint(object):
    """Backward of training-mode batch normalisation in closed form:

        dbeta = sum(d), dgamma = sum(d * xhat), dx = gamma * rstd * (d - dbeta/m - xhat * dgamma/m)

    with xhat = (x - mean) * rstd and m elements per channel: one pass with two reductions and one
    elementwise pass, instead of the chain of dependent reductions that differentiating the
    two-pass variance op by op gives (six passes over x)."""

    def __init__(self, flat, gamma, beta, xmean, rstd, out_axes):
        self.flat, self.gamma, self.beta = flat, gamma, beta
        self.xmean, self.rstd, self.out_axes = xmean, rstd, out_axes

    def generate_adjoints(self, add_delta, adjoints, delta):
        d = ng.flatten(ng.axes_with_order(delta, ng.unflatten(self.flat).axes), self.flat.axes) \
            if not delta.axes.is_equal_set(self.flat.axes) else ng.axes_with_order(delta, self.flat.axes)
        m = float((self.flat.axes - self.out_axes).size)
        xhat = (self.flat - self.xmean) * self.rstd
        dbeta = ng.sum(d, out_axes=self.out_axes)
        dgamma = ng.sum(d * xhat, out_axes=self.out_axes)
        dx = (self.gamma * self.rstd) * (d - dbeta * (1.0 / m) - xhat * (dgamma * (1.0 / m)))
        add_delta(adjoints, self.flat, dx)
        if isinstance(self.gamma, ng.TensorOp):
            add_delta(adjoints, self.gamma, dgamma)
        if isinstance(self.beta, ng.TensorOp):
            add_delta(adjoints, self.beta, dbeta)


# ---- a training step out of a cost (ngraph/frontends/neon/optimizer.py:50-120, 159-209) -------
def clip_gradient_norm(grad_list, clip_norm=None):
    """Factor <= 1 that brings the joint L2 norm of the gradients down to clip_norm."""
    if clip_norm is None:
        return 1
    s = None
    for g in grad_list:
        term = ng.squared_L2(g, out_axes=None)
        s = term if s is None else s + term
    return clip_norm / ng.maximum(ng.sqrt(s), clip_norm)


def clip_gradient_value(grad, clip_value=None):
    if clip_value is None:
        return grad
    return ng.minimum(ng.maximum(grad, -abs(clip_value)), abs(clip_value))


def clip_weight_value(weight, clip_value=None, min_value_override=None):
    if clip_value is None:
        return weight
    if min_value_override is None:
        min_value_override = -abs(clip_value)
    return ng.minimum(ng.maximum(weight, min_value_override), abs(clip_value))


def trainable_variables(op):
    """The trainable variables `op` is computed from, in graph order."""
    from ngraph_hip.op_graph.op_graph import Op, AssignableTensorOp
    found = []
    for o in Op.ordered_ops([op]):
        for s in o.states_read:
            if isinstance(s, AssignableTensorOp) and s.is_trainable and s not in found:
                found.append(s)
    return found


class Optimizer(object):
    """What the reference's LearningRateOptimizer.__call__ does with a cost: gradients of the
    summed cost divided by the batch size, optional clipping, one update per variable; the
    returned op runs gradients, updates and weight clipping in that order."""

    gradient_clip_norm = None
    gradient_clip_value = None
    weight_clip_value = None

    def minimize(self, cost_func, variables=None):
        batch_cost = ng.sum(cost_func, out_axes=())
        batch_axis = cost_func.axes.batch_axis()
        batch_size = 1 if batch_axis is None else batch_axis.length
        if variables is None:
            variables = trainable_variables(batch_cost)
        self.prepare()
        grads = [ng.deriv(batch_cost, v) / batch_size for v in variables]
        scale_factor = clip_gradient_norm(grads, self.gradient_clip_norm)
        grads = [clip_gradient_value(g, self.gradient_clip_value) for g in grads]
        updates = []
        for variable, grad in zip(variables, grads):
            out = self.variable_update(variable, grad, scale_factor)
            updates.append(out[0] if isinstance(out, tuple) else out)
        steps = list(updates)
        if self.weight_clip_value is not None:
            steps += [ng.assign(v, clip_weight_value(v, self.weight_clip_value)) for v in variables]
        return ng.sequential(steps + [batch_cost])

    def prepare(self):
        pass

    def _set_clipping(self, gradient_clip_norm=None, gradient_clip_value=None, weight_clip_value=None):
        self.gradient_clip_norm = gradient_clip_norm
        self.gradient_clip_value = gradient_clip_value
        self.weight_clip_value = weight_clip_value


class Adam(Optimizer):
    """Adam learning rule; `__call__` advances t, `variable_update` builds one update."""

    def __init__(self, learning_rate=1e-3, beta_1=0.9, beta_2=0.999, epsilon=1e-8, **clipping):
        self._set_clipping(**clipping)
        self.lrate = learning_rate
        self.beta_1 = ng.constant(beta_1, dtype=np.float32)
        self.beta_2 = ng.constant(beta_2, dtype=np.float32)
        self.epsilon = epsilon
        self.t = ng.persistent_tensor(axes=(), initial_value=0)
        self.step = None
        self.ell = None

    def prepare(self):
        if self.ell is None:
            self()

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


class GradientDescentMomentum(Optimizer):
    """SGD with momentum, weight decay, optional Nesterov step and the Kahan-compensated
    parameter update of frontends/neon/optimizer.py:285-310."""

    def __init__(self, learning_rate, momentum_coef=0.0, wdecay=0.0, nesterov=False, **clipping):
        self._set_clipping(**clipping)
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


class RMSProp(Optimizer):
    """frontends/neon/optimizer.py:370-383."""

    def __init__(self, decay_rate=0.95, learning_rate=2e-3, epsilon=1e-6, wdecay=0.0, momentum_coef=0.0, **clipping):
        self._set_clipping(**clipping)
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


class Adagrad(Optimizer):
    """frontends/neon/optimizer.py:533-542."""

    def __init__(self, learning_rate=0.01, epsilon=1e-6, **clipping):
        self._set_clipping(**clipping)
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
