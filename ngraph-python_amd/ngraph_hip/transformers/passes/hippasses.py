"""Graph passes of the HIP backend itself, run after the front's own (SimplePrune):

* TensorSizeFold      TensorSizeOp becomes a constant;
* ConstantFoldPass    elementwise ops on scalar constants are evaluated at transform time;
* ReductionLayoutPass a reduction whose reduced axes do not form one strided axis is taken in
                      steps over groups of axes that do, or (argmax / argmin, flex) gets a copy
                      of its operand in (reduced..., kept...) order -- where the reference
                      inserts a DimshuffleOp (gpulayout.py:861-979, layout_common.py:347-378).

They use the graph package only through the names imported below, so the same source serves
the graph front of this repository and the real `ngraph` package (ngraph_hip/plugin.py).
"""
from __future__ import division
import numpy as np

from ngraph_hip.op_graph.op_graph import TensorSizeOp, ContiguousOp, ReductionOp, constant, axes_with_order
from ngraph_hip.transformers.passes.passes import PeepholeGraphPass


def _scalar_const(x):
    """The Python value of a scalar constant op (seen through reads), or None."""
    if x.is_scalar and x.is_constant:
        return float(np.asarray(x.const).reshape(()))
    return None


def _td(op):
    """The tensor description of `op` in this backend's conventions (element strides); the
    plug-in for the real package replaces `_adapt_td`, which is the identity here."""
    return _adapt_td(op.tensor_description())


def _adapt_td(td):
    return td


class TensorSizeFold(PeepholeGraphPass):
    """TensorSizeOp is known at transform time: make it a constant.

    The reference backends fill a scalar tensor with `reduction_axes.size`
    (gputransform.py:444-447, cputransform.py:759-761); a constant gives the
    same value and lets it travel as a kernel argument.
    """

    def visit(self, op, *args):
        if isinstance(op, TensorSizeOp):
            self.replace_op(op, constant(float(op.reduction_axes.size)))


def axes_merge_to_one(td, axes):
    """Can `axes` of the view `td` be walked as ONE strided dimension?"""
    dims = [(a.length, td.full_strides[td.axes.index(a)]) for a in axes if a.length != 1]
    dims.sort(key=lambda d: -d[1])
    for (n0, s0), (n1, s1) in zip(dims[:-1], dims[1:]):
        if s0 != s1 * n1:
            return False
    return True


def strided_axis_groups(td, axes):
    """`axes` of the view `td` partitioned into groups that can each be walked as one strided
    dimension (outermost group first)."""
    dims = sorted(((td.full_strides[td.axes.index(a)], a) for a in axes if a.length != 1), key=lambda d: -d[0])
    groups = []
    for stride, axis in dims:
        if groups and groups[-1][1] == stride * axis.length:
            groups[-1][0].append(axis)
            groups[-1][1] = stride
        else:
            groups.append([[axis], stride])
    groups = [g[0] for g in groups]
    unit = [a for a in axes if a.length == 1]
    if unit:
        groups = ([groups[0] + unit] + groups[1:]) if groups else [unit]
    return groups


class ReductionLayoutPass(PeepholeGraphPass):
    """Reductions need their reduced axes to form one strided axis.

    When they do not, the reference copies the operand into (reduced..., kept...) order with a
    DimshuffleOp (gpulayout.py:861-979, layout_common.py:347-378): a full extra read and write
    of the operand.  With `split`, a sum, product, maximum or minimum is instead taken group by
    group of axes that do form one strided axis, the largest group first -- sum over (N, HW) of
    an [N, C, HW] tensor becomes sum over N of (sum over HW): one pass over the operand and a
    small second reduction, no copy.  The result is the same reduction in another association
    order; argmax / argmin (whose results are positions in the original axis), and storage
    types that round every stored intermediate (`split=False`), keep the copy.
    """

    _SPLITTABLE = ("Sum", "Prod", "Max", "Min")

    def __init__(self, split=True, **kwargs):
        super(ReductionLayoutPass, self).__init__(**kwargs)
        self.split = split

    def visit(self, op, *args):
        if not isinstance(op, ReductionOp) or len(op.reduction_axes) < 2:
            return
        x, = args
        if axes_merge_to_one(_td(x), op.reduction_axes):
            return
        if self.split and type(op).__name__ in self._SPLITTABLE:
            groups = strided_axis_groups(_td(x), op.reduction_axes)
            if len(groups) > 1:
                first = max(groups, key=lambda g: int(np.prod([a.length for a in g])))
                rest = [a for a in op.reduction_axes if a not in first]
                inner = type(op)(x, reduction_axes=first, dtype=op.dtype)
                # (the outer reduction is visited in the next sweep and split again if need be)
                self.replace_op(op, type(op)(inner, reduction_axes=rest, dtype=op.dtype))
                return
        order = op.reduction_axes + (x.axes - op.reduction_axes)
        new_x = ContiguousOp(axes_with_order(x, order))
        self.replace_op(op, type(op)(new_x, reduction_axes=op.reduction_axes, dtype=op.dtype))


class ConstantFoldPass(PeepholeGraphPass):
    """Elementwise ops on scalar constants are evaluated at transform time.

    Such subgraphs ((1 - beta_1), lr * 2, ...) would otherwise each cost a kernel launch per
    call.  The value is computed in float32 with the NumPy ufunc of the same name, which is
    what the per-op CPU path does with the same operands (cputransform.py:512-761).
    """

    _UNARY = {"NegativeOp": np.negative, "AbsoluteOp": np.abs, "SqrtOp": np.sqrt, "ExpOp": np.exp,
              "LogOp": np.log, "ReciprocalOp": np.reciprocal, "SquareOp": np.square,
              "TanhOp": np.tanh, "SignOp": np.sign, "SinOp": np.sin, "CosOp": np.cos}
    _BINARY = {"Add": np.add, "Subtract": np.subtract, "Multiply": np.multiply,
               "Divide": np.divide, "Power": np.power, "Maximum": np.maximum,
               "Minimum": np.minimum, "FloorDivide": np.floor_divide, "Mod": np.mod}

    def visit(self, op, *args):
        name = type(op).__name__
        if name not in self._UNARY and name not in self._BINARY:
            return
        if op.dtype != np.dtype(np.float32):
            return
        if name in self._UNARY and len(args) == 1:
            c = _scalar_const(args[0])
            if c is not None:
                with np.errstate(all="ignore"):
                    val = self._UNARY[name](np.float32(c), dtype=np.float32)
                self.replace_op(op, constant(float(val), op.axes))
        elif name in self._BINARY and len(args) == 2:
            cx, cy = _scalar_const(args[0]), _scalar_const(args[1])
            if cx is not None and cy is not None:
                with np.errstate(all="ignore"):
                    val = self._BINARY[name](np.float32(cx), np.float32(cy), dtype=np.float32)
                self.replace_op(op, constant(float(val), op.axes))
