"""Reverse-mode differentiation of the elementwise / reduction / view part of the graph.

`deriv(dependent, independent, error)` builds, out of ordinary ops, the graph that computes
d dependent / d independent applied to `error` (op_graph.py:1120-1183 `adjoints` and
`generate_add_delta`, :4268-4314 `DerivOp`).  The backward graph consists of the same
elementwise ops, reductions and views as the forward one, so the fusion planner treats it like
any other group of ops.

Each rule below restates the `generate_adjoints` of the reference's op of the same name
(op_graph.py:2903-3482 elementwise, :3935-3990 reductions, :1741-2284 views).  Ops without a
rule contribute no gradient, as in the reference (comparisons, sign, argmax, one-hot, sizes,
random fills); dense ops are not part of this package.
"""
from __future__ import division

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.op_graph.axes import make_axes


def _key(op):
    """Adjoints are kept per tensor: a read of a variable stands for the variable."""
    op = op.forwarded
    if isinstance(op, og.ValueOp):
        return op.tensor.forwarded
    return op


def _add_delta(adjoints, x, delta):
    x = x.forwarded
    delta = og.as_op(delta)
    if not x.axes.is_equal_set(delta.axes):
        raise ValueError("delta axes {} do not match adjoint axes {}".format(delta.axes, x.axes))
    key = _key(x)
    if key in adjoints:
        adjoints[key] = delta + adjoints[key]
    else:
        adjoints[key] = delta


class UnsliceOp(og.SequentialOp):
    """The reverse of a slice: zeros in the shape of `axes` with x in the slice
    (op_graph.py:2737-2765)."""

    def __init__(self, x, slices, axes, **kwargs):
        super(UnsliceOp, self).__init__(**kwargs)
        temp = og.temporary(axes=axes, dtype=x.dtype).named("unslice")
        window = og.tensor_slice(temp, slices, axes=x.axes)
        self.ops = [og.Fill(temp, 0), og.assign(window, x), og.value_of(temp)]


def _unslice(x, slices, axes):
    return UnsliceOp(x, slices, axes).value_tensor


RULES = {}


def _rule(*names):
    def register(fn):
        for name in names:
            RULES[name] = fn
        return fn
    return register


# ---- elementwise ---------------------------------------------------------------------------
@_rule("NegativeOp")
def _neg(op, adjoints, delta, x):
    _add_delta(adjoints, x, -delta)


@_rule("AbsoluteOp")
def _abs(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.sign(x) * delta)


@_rule("SinOp")
def _sin(op, adjoints, delta, x):
    _add_delta(adjoints, x, delta * og.cos(x))


@_rule("CosOp")
def _cos(op, adjoints, delta, x):
    _add_delta(adjoints, x, -delta * og.sin(x))


@_rule("TanhOp")
def _tanh(op, adjoints, delta, x):
    _add_delta(adjoints, x, delta * (1.0 - op * op))


@_rule("ExpOp")
def _exp(op, adjoints, delta, x):
    _add_delta(adjoints, x, delta * op)


@_rule("LogOp")
def _log(op, adjoints, delta, x):
    _add_delta(adjoints, x, delta / x)


@_rule("ReciprocalOp")
def _rcp(op, adjoints, delta, x):
    _add_delta(adjoints, x, -op * op * delta)


@_rule("SquareOp")
def _sqr(op, adjoints, delta, x):
    _add_delta(adjoints, x, 2.0 * delta * x)


@_rule("SqrtOp")
def _sqrt(op, adjoints, delta, x):
    _add_delta(adjoints, x, 0.5 * delta / op)


@_rule("SigmoidAtomicOp")
def _sigmoid(op, adjoints, delta, x):
    _add_delta(adjoints, x, delta * op * (1.0 - op))


@_rule("Add")
def _add(op, adjoints, delta, x, y):
    _add_delta(adjoints, x, delta)
    _add_delta(adjoints, y, delta)


@_rule("Subtract")
def _sub(op, adjoints, delta, x, y):
    _add_delta(adjoints, x, delta)
    _add_delta(adjoints, y, -delta)


@_rule("Multiply")
def _mul(op, adjoints, delta, x, y):
    _add_delta(adjoints, x, delta * y)
    _add_delta(adjoints, y, x * delta)


@_rule("Divide")
def _div(op, adjoints, delta, x, y):
    _add_delta(adjoints, x, delta * op / x)
    _add_delta(adjoints, y, -delta * op / y)


@_rule("Maximum")
def _maximum(op, adjoints, delta, x, y):
    _add_delta(adjoints, x, og.greater(x, y) * delta)
    _add_delta(adjoints, y, og.greater(y, x) * delta)


@_rule("Minimum")
def _minimum(op, adjoints, delta, x, y):
    _add_delta(adjoints, x, og.less(x, y) * delta)
    _add_delta(adjoints, y, og.less(y, x) * delta)


@_rule("Power")
def _pow(op, adjoints, delta, x, y):
    _add_delta(adjoints, x, delta * y * op / x)
    _add_delta(adjoints, y, delta * op * og.log(x))


# ---- reductions ----------------------------------------------------------------------------
@_rule("Sum")
def _sum(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.broadcast(delta, x.axes))


@_rule("Max", "Min")
def _extremum(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.equal(x, op) * delta)


@_rule("Prod")
def _prod(op, adjoints, delta, x):
    # d prod / dx_i = prod of the others; formed as prod / x_i, so zeros in x are not handled
    # (the reference treats them separately, op_graph.py:3959-3987)
    _add_delta(adjoints, x, og.broadcast(op * delta, x.axes) / x)


# ---- views ---------------------------------------------------------------------------------
@_rule("BroadcastOp")
def _broadcast(op, adjoints, delta, x):
    dx = og.sum(delta, reduction_axes=delta.axes - x.axes)
    _add_delta(adjoints, x, og.axes_with_order(dx, x.axes))


@_rule("ExpandDims")
def _expand_dims(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.sum(delta, reduction_axes=delta.axes - x.axes))


@_rule("ReorderAxes")
def _reorder(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.axes_with_order(delta, x.axes))


@_rule("Transpose")
def _transpose(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.Transpose(delta))


@_rule("AxesCastOp")
def _cast(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.cast_axes(delta, x.axes))


@_rule("Flatten")
def _flatten(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.unflatten(delta, axes=x.axes))


@_rule("Unflatten")
def _unflatten(op, adjoints, delta, x):
    _add_delta(adjoints, x, og.flatten(delta, axes=x.axes))


@_rule("TensorSliceOp")
def _slice(op, adjoints, delta, x):
    _add_delta(adjoints, x, _unslice(delta, op.slices, x.axes))


@_rule("ContiguousOp")
def _contiguous(op, adjoints, delta, x):
    _add_delta(adjoints, x, delta)


def adjoints_of(dependent, error):
    """{tensor: d dependent / d tensor applied to error} for every tensor `dependent` is
    computed from (op_graph.py:1120-1164)."""
    dependent = dependent.forwarded
    adjoints = {_key(dependent): error}
    processed = set()
    for o in reversed(og.Op.ordered_ops([dependent])):
        if not o.is_tensor_op:
            continue
        key = _key(o)
        if key in processed or key not in adjoints:
            continue
        processed.add(key)
        target = key if isinstance(o, og.ValueOp) else o
        adjoint = adjoints[key]
        if getattr(target, "scale", None) is not None:
            adjoint = adjoint * target.scale
        # a composite may differentiate itself as a whole (op_graph.py:1153-1160 deriv_handler):
        # sigmoid, softmax, the cross entropies of either, batch normalisation
        # (the value of a stack / concat may be the plain read of its storage: look on the read too)
        handler = getattr(o, "deriv_handler", None) or getattr(target, "deriv_handler", None)
        if handler is not None and handler is not target:
            handler.generate_adjoints(_add_delta, adjoints, adjoint)
            continue
        rule = RULES.get(type(target).__name__)
        if rule is not None:
            rule(target, adjoints, adjoint, *[a.forwarded for a in target.args])
    return adjoints


def deriv(dependent, independent, error=None):
    """The op computing [d dependent / d independent](error); it has independent's axes.
    `error` defaults to the scalar 1: a tensor-valued dependent needs an explicit error."""
    dependent, independent = og.as_op(dependent), og.as_op(independent)
    # One backward graph per (dependent, error): derivatives with respect to several tensors share
    # it (there is no common-subexpression elimination to merge separate copies later).  The default
    # error is one constant per dependent for the same reason (op_graph.py:4275-4282); being a
    # scalar, it only suits a scalar dependent.
    cache = dependent.forwarded.__dict__.setdefault("_adjoint_cache", {})
    if error is None:
        if "one" not in cache:
            cache["one"] = og.constant(1.0)
        error = cache["one"]
    error = og.as_op(error)
    if not error.axes.is_equal_set(dependent.axes):
        raise ValueError("Dependent and error must have the same set of axes")
    error_key = id(_key(error))          # a placeholder is wrapped anew at every use
    if error_key not in cache:
        cache[error_key] = (error, adjoints_of(dependent, error))
    adjoints = cache[error_key][1]
    key = _key(independent)
    if key not in adjoints:
        return og.constant(0, independent.axes)       # not connected (op_graph.py:4286-4287)
    adjoint = adjoints[key]
    return og.axes_with_order(og.broadcast(adjoint, make_axes(independent.axes)), independent.axes)
