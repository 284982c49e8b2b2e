"""`cpu_bound`: float64 evaluation of an op graph with a running forward error bound.
ORACLE ONLY (test infrastructure).

For graphs whose float32 result is ill conditioned (cancellation, long products, chains of
exponentials) two correct float32 evaluations -- the NumPy statements of the reference CPU
transformer (ngraph/transformers/cputransform.py:512-761) and the device kernels -- differ by
more than any fixed tolerance.  This evaluator arbitrates: it runs the same (pruned) graph in
float64 and carries, element by element, a bound on how far ANY float32 evaluation may be
from that value when every op is computed from the float32 results before it and rounded

* once (unit roundoff u = 2^-24) for +, -, *, /, sqrt, reciprocal, square;
* to within `TRANSCENDENTAL_ULPS` units in the last place for exp, log, tanh, sin, cos, pow,
  sigmoid (the device is tested to stay within 2 ulp; NumPy's float32 loops are within 3);
* a sum over n elements in any order: min(n, 8 sqrt(n)) u sum|x_i| -- the probabilistic bound
  of a serial sum, which is what NumPy does across a strided axis (the worst case n u says
  nothing at n ~ 10^5; trees are tighter than either);
* a comparison, sign, argmax or argmin whose operands are closer than their bounds may come
  out either way: the bound becomes infinite there ("undecided"), and a test leaves such
  elements out.

Input errors propagate through exact interval images for monotone functions and through
first-order terms with the second-order product kept for multiplications.  The bound describes
op-by-op evaluation; fused kernels that re-associate (one-pass moments) stay within it in
practice because the sum bound is that of a serial sum.

Nothing in the product imports this module.
"""
from __future__ import division

import numpy as np

from ngraph_hip.op_graph import op_graph as og
from oracle.cpu_transformer import (NumpyTransformer, NumpyDeviceBufferStorage, NumpyDeviceTensor,
                                    numpy_call_name)
from oracle import numpy_ops

f64 = np.float64
U = 2.0 ** -24                      # float32 unit roundoff
TINY = 2.0 ** -149                  # smallest float32 subnormal: absolute rounding floor
TRANSCENDENTAL_ULPS = 4
FLT_MAX = float(np.finfo(np.float32).max)


def _rounded(v, ulps=0.5):
    """Bound of the rounding error of a float32 result near v: `ulps` units in the last place
    (one ulp <= 2 u |v|)."""
    return 2.0 * ulps * U * np.abs(v) + TINY


def _image(fn, x, ex):
    """max |fn(x +- ex) - fn(x)| for a function monotone between x - ex and x + ex; infinite
    where an end point leaves the domain."""
    with np.errstate(all="ignore"):
        v = fn(x)
        d = np.maximum(np.abs(fn(x + ex) - v), np.abs(fn(x - ex) - v))
    return np.where(np.isfinite(d), d, np.inf)


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def _undecided(mask):
    return np.where(mask, np.inf, 0.0)


# name -> (value function, error function(x, ex, v))
UNARY = {
    "abs": (np.abs, lambda x, ex, v: ex),
    "neg": (np.negative, lambda x, ex, v: ex),
    "sqrt": (np.sqrt, lambda x, ex, v: _image(np.sqrt, x, ex) + _rounded(v)),
    "sqr": (np.square, lambda x, ex, v: 2 * np.abs(x) * ex + ex * ex + _rounded(v)),
    "exp": (np.exp, lambda x, ex, v: _image(np.exp, x, ex) + _rounded(v, TRANSCENDENTAL_ULPS)),
    "exp2": (np.exp2, lambda x, ex, v: _image(np.exp2, x, ex) + _rounded(v, TRANSCENDENTAL_ULPS)),
    "log": (np.log, lambda x, ex, v: _image(np.log, x, ex) + _rounded(v, TRANSCENDENTAL_ULPS)),
    "log2": (np.log2, lambda x, ex, v: _image(np.log2, x, ex) + _rounded(v, TRANSCENDENTAL_ULPS)),
    "rcp": (np.reciprocal,
            lambda x, ex, v: np.where(np.abs(x) > ex, _image(np.reciprocal, x, ex), np.inf) + _rounded(v)),
    "tanh": (np.tanh, lambda x, ex, v: _image(np.tanh, x, ex) + _rounded(v, TRANSCENDENTAL_ULPS)),
    "sig": (_sigmoid, lambda x, ex, v: _image(_sigmoid, x, ex) + _rounded(v, 2 * TRANSCENDENTAL_ULPS)),
    "sin": (np.sin, lambda x, ex, v: ex + _rounded(v, TRANSCENDENTAL_ULPS)),
    "cos": (np.cos, lambda x, ex, v: ex + _rounded(v, TRANSCENDENTAL_ULPS)),
    "sgn": (np.sign, lambda x, ex, v: _undecided((np.abs(x) <= ex) & (ex > 0))),
    "assign": (lambda x: x, lambda x, ex, v: ex),
}


def _div_err(x, y, ex, ey, v):
    with np.errstate(all="ignore"):
        e = (ex + np.abs(v) * ey) / (np.abs(y) - ey)
    return np.where(np.abs(y) > ey, e, np.inf) + _rounded(v)


def _compare_err(x, y, ex, ey, v):
    return _undecided((np.abs(x - y) <= ex + ey) & (ex + ey > 0))


def _corner_err(fn, ulps):
    """Deviation over the corners of the operand box, for functions monotone in each operand
    over the box; infinite when a corner leaves the domain."""
    def err(x, y, ex, ey, v):
        with np.errstate(all="ignore"):
            d = np.zeros(np.broadcast(x, y).shape)
            for sx in (-1.0, 1.0):
                for sy in (-1.0, 1.0):
                    d = np.maximum(d, np.abs(fn(x + sx * ex, y + sy * ey) - v))
        d = np.where(np.isfinite(d), d, np.inf)
        exact = (ex == 0) & (ey == 0)
        return np.where(exact, 0.0, d) + _rounded(v, ulps)
    return err


def _floor_err(fn):
    """floor_divide and mod jump where x / y crosses an integer."""
    def err(x, y, ex, ey, v):
        with np.errstate(all="ignore"):
            qs = [np.floor((x + sx * ex) / (y + sy * ey)) for sx in (-1.0, 1.0) for sy in (-1.0, 1.0)]
            jump = (np.minimum.reduce(qs) != np.maximum.reduce(qs)) | (np.abs(y) <= ey)
        return np.where(jump, np.inf, _corner_err(fn, 1.0)(x, y, ex, ey, v))
    return err


BINARY = {
    "add": (np.add, lambda x, y, ex, ey, v: ex + ey + _rounded(v)),
    "sub": (np.subtract, lambda x, y, ex, ey, v: ex + ey + _rounded(v)),
    "mul": (np.multiply, lambda x, y, ex, ey, v: np.abs(x) * ey + np.abs(y) * ex + ex * ey + _rounded(v)),
    "div": (np.divide, _div_err),
    "int_div": (np.floor_divide, _floor_err(np.floor_divide)),
    "mod": (np.mod, _floor_err(np.mod)),
    "pow": (np.power, _corner_err(np.power, TRANSCENDENTAL_ULPS)),
    "minimum": (np.minimum, lambda x, y, ex, ey, v: np.maximum(ex, ey)),
    "maximum": (np.maximum, lambda x, y, ex, ey, v: np.maximum(ex, ey)),
    "eq": (np.equal, _compare_err), "ne": (np.not_equal, _compare_err),
    "lt": (np.less, _compare_err), "le": (np.less_equal, _compare_err),
    "gt": (np.greater, _compare_err), "ge": (np.greater_equal, _compare_err),
}


def _count(x, axis):
    axes = (axis,) if isinstance(axis, int) else tuple(axis)
    n = 1
    for a in axes:
        n *= x.shape[a]
    return n


def _sum_err(x, ex, axis, v):
    n = _count(x, axis)
    return ex.sum(axis=axis) + min(n, 8.0 * np.sqrt(n)) * U * (np.abs(x) + ex).sum(axis=axis) + TINY


def _prod_err(x, ex, axis, v):
    n = _count(x, axis)
    with np.errstate(all="ignore"):
        rel = np.where(ex > 0, ex / (np.abs(x) - ex), 0.0)
        rel = np.where((ex > 0) & (np.abs(x) <= ex), np.inf, rel)
        total = np.expm1(np.log1p(rel).sum(axis=axis) + n * U)
    return np.abs(v) * total + TINY


def _extreme_err(x, ex, axis, v):
    return ex.max(axis=axis)


REDUCE = {"sum": (np.sum, _sum_err), "prod": (np.prod, _prod_err),
          "max": (np.max, _extreme_err), "min": (np.min, _extreme_err)}


def _arg_err(name, x, ex, axis):
    """A position is decided when the winner beats every other element by more than both
    bounds (exact ties go to the first index in every implementation, cputransform.py:521-527)."""
    sign = 1.0 if name == "argmax" else -1.0
    s = sign * x
    pos = s.argmax(axis=axis)
    best_low = np.take_along_axis(s - ex, np.expand_dims(pos, axis), axis)
    rivals = (s + ex >= best_low) & (ex + np.take_along_axis(ex, np.expand_dims(pos, axis), axis) > 0)
    idx = np.arange(x.shape[axis]).reshape([-1 if i == axis else 1 for i in range(x.ndim)])
    rivals = rivals & (idx != np.expand_dims(pos, axis))
    return _undecided(rivals.any(axis=axis))


class BoundDeviceBufferStorage(NumpyDeviceBufferStorage):
    """Two float64 arrays per base tensor: the value and the bound."""

    def __init__(self, transformer, bytes, dtype, **kwargs):
        super(BoundDeviceBufferStorage, self).__init__(transformer, bytes, dtype, **kwargs)
        n = self.data.size
        self.data = np.zeros(n, dtype=f64)
        self.err = np.zeros(n, dtype=f64)

    def create_device_tensor(self, tensor_description):
        return BoundDeviceTensor(self.transformer, self, tensor_description)


class BoundDeviceTensor(NumpyDeviceTensor):
    def _strided(self, base):
        td = self.tensor_description
        return np.lib.stride_tricks.as_strided(
            base[td.offset:], shape=td.shape,
            strides=tuple(s * base.dtype.itemsize for s in td.full_strides), writeable=True)

    @property
    def view(self):
        return self._strided(self.device_buffer.data)

    @property
    def err_view(self):
        return self._strided(self.device_buffer.err)

    def __setitem__(self, key, value):
        # what the host writes is float32 data, exactly known
        key = key if key is not Ellipsis else ()
        self.view.__setitem__(key, np.asarray(value, dtype=np.float32).astype(f64))
        self.err_view.__setitem__(key, 0.0)


class BoundTransformer(NumpyTransformer):
    transformer_name = "cpu_bound"

    def device_buffer_storage(self, bytes, dtype, name):
        return BoundDeviceBufferStorage(self, bytes, dtype, name="a_" + name)

    def _pair(self, op):
        t = self.get_tensor_description_tensor_view(op.forwarded.tensor_description())
        return t.view, t.err_view

    def error_bound(self, op):
        """The bound that belongs to the value the last call left in `op`'s tensor."""
        return np.array(self._pair(op)[1], copy=True)

    def _step(self, op):
        pair = self._pair
        name = numpy_call_name(op)

        def put(out_op, v, e):
            ov, oe = pair(out_op)
            ov[()] = v
            oe[()] = np.where(np.isnan(e), np.inf, e)

        if isinstance(op, og.AssignOp):
            return lambda: put(op.args[0], *pair(op.args[1]))
        if isinstance(op, og.Fill):
            return lambda: put(op.args[0], f64(np.float32(op.scalar)), 0.0)
        if isinstance(op, og.TensorSizeOp):
            return lambda: put(op, f64(op.reduction_axes.size), 0.0)
        if isinstance(op, og.ContiguousOp):
            return lambda: put(op, *pair(op.args[0]))
        if isinstance(op, og.OneHotOp):
            def onehot():
                x, ex = pair(op.args[0])
                n = pair(op)[0].shape[0]
                put(op, np.eye(n)[:, x.astype(np.int32)], _undecided(ex > 0)[np.newaxis])
            return onehot
        if isinstance(op, og.RngOp):
            return lambda: put(op, 0.0, np.inf)
        if isinstance(op, og.LookupTableOp):
            def lookup():
                (lut, elut), (idx, eidx) = pair(op.args[0]), pair(op.args[1])
                where = idx.astype(int)
                e = elut.take(where, op.lut_axis)
                put(op, lut.take(where, op.lut_axis), np.where(np.any(eidx > 0), np.inf, e))
            return lookup
        if isinstance(op, og.ReductionOp):
            x_axes = op.args[0].forwarded.axes
            np_axis = tuple(x_axes.index(a) for a in op.reduction_axes)
            np_axis = np_axis[0] if len(np_axis) == 1 else np_axis

            def reduce():
                x, ex = pair(op.args[0])
                with np.errstate(all="ignore"):
                    if np_axis == ():
                        put(op, *((0.0, 0.0) if name in ("argmax", "argmin") else (x, ex)))
                    elif name in ("argmax", "argmin"):
                        if isinstance(np_axis, tuple):
                            raise NotImplementedError("argmax over several axes")
                        put(op, getattr(np.ndarray, name)(x, axis=np_axis), _arg_err(name, x, ex, np_axis))
                    else:
                        fn, err = REDUCE[name]
                        v = fn(x, axis=np_axis)
                        put(op, v, err(x, ex, np_axis, v))
            return reduce
        if name in UNARY:
            fn, err = UNARY[name]

            def unary():
                x, ex = pair(op.args[0])
                with np.errstate(all="ignore"):
                    v = fn(x)
                    put(op, v, err(x, ex, v))
            return unary
        if name in BINARY:
            fn, err = BINARY[name]

            def binary():
                (x, ex), (y, ey) = pair(op.args[0]), pair(op.args[1])
                with np.errstate(all="ignore"):
                    v = fn(x, y).astype(f64)
                    put(op, v, err(x, y, ex, ey, v))
            return binary
        raise ValueError("bound evaluator has no rule for op {}".format(op))


def within_bound(result, value, bound, rtol, atol):
    """Element-wise: is the float32 `result` within tolerance + bound of the float64 `value`?
    Elements whose bound is infinite (undecided comparisons upstream) or whose value is outside
    float32's range count as within."""
    result = np.asarray(result, dtype=f64)
    free = ~np.isfinite(bound) | ~np.isfinite(value) | (np.abs(value) + bound >= FLT_MAX)
    with np.errstate(all="ignore"):
        ok = np.abs(result - value) <= atol + rtol * np.abs(value) + bound
    return ok | free


assert set(UNARY) >= set(numpy_ops.UNARY) and set(BINARY) == set(numpy_ops.BINARY)
