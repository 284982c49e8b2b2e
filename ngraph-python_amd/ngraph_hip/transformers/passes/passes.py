"""Graph passes run before lowering.

Counterparts of ngraph/transformers/passes/passes.py for the op set of this
path: the pass driver (passes.py:35-120), `replace_op` with axes repair, and
the `SimplePrune` algebra (passes.py:499-628) that changes which ops reach the
kernels (x*1, x*0, x*-1, x+0, constant sum/prod, log(exp x), -const).
"""
from __future__ import division
import numpy as np

from ngraph_hip.op_graph.op_graph import (
    Op, NegativeOp, Multiply, Add, Sum, Prod, LogOp, ExpOp, Divide, TensorSizeOp, ContiguousOp,
    BroadcastOp, constant, negative, broadcast, axes_with_order, as_op, TensorOp)


class GraphPass(object):
    def wrapped_do_pass(self, **kwargs):
        self.do_pass(**kwargs)

    def do_pass(self, ops, **kwargs):
        raise NotImplementedError


class PeepholeGraphPass(GraphPass):
    """Visit every op in dependency order; replacements apply after each sweep."""

    def do_pass(self, ops, **kwargs):
        has_work = True
        while has_work:
            self.replacement_list = []
            for op in Op.ordered_ops(ops):
                op = op.forwarded
                self.visit(op, *self.op_args(op))
            for old, rep in self.replacement_list:
                old.forwarded.forward = rep.forwarded if rep.forwarded is not old.forwarded else None
            has_work = len(self.replacement_list) > 0

    @staticmethod
    def op_arg(op, n):
        return op.args[n].forwarded

    @staticmethod
    def op_args(op):
        return tuple(a.forwarded for a in op.args)

    def replace_op(self, op, replacement):
        """Use `replacement` wherever `op` was used; its axes are repaired to op's (passes.py:86-120)."""
        replacement = as_op(replacement)
        if isinstance(op, TensorOp) and replacement.axes != op.axes:
            replacement = axes_with_order(broadcast(replacement, op.axes), op.axes)
        self.replacement_list.append((op, replacement))

    def visit(self, op, *args):
        pass


def _scalar_const(x):
    """The Python value of a scalar constant op (seen through reads), or None."""
    if x.is_scalar and x.is_constant:
        return float(np.asarray(x.const).reshape(()))
    return None


class SimplePrune(PeepholeGraphPass):
    """Algebraic simplifications (passes.py:499-628)."""

    def visit(self, op, *args):
        if isinstance(op, NegativeOp):
            x, = args
            c = _scalar_const(x)
            if c is not None:
                self.replace_op(op, constant(-c, op.axes))
        elif isinstance(op, Multiply):
            x, y = args
            rep = None
            cx, cy = _scalar_const(x), _scalar_const(y)
            if cx is not None:
                if cx == 0:
                    rep = x
                elif cx == 1:
                    rep = y
                elif cx == -1:
                    rep = negative(y)
            elif cy is not None:
                if cy == 0:
                    rep = y
                elif cy == 1:
                    rep = x
                elif cy == -1:
                    rep = negative(x)
            if rep is not None:
                self.replace_op(op, rep)
        elif isinstance(op, Add):
            x, y = args
            rep = None
            cx, cy = _scalar_const(x), _scalar_const(y)
            if cx is not None:
                if cx == 0:
                    rep = y
            elif cy is not None:
                if cy == 0:
                    rep = x
            elif isinstance(y, ContiguousOp) and isinstance(self.op_arg(y, 0), BroadcastOp):
                inner = self.op_arg(self.op_arg(y, 0), 0)
                if _scalar_const(inner) == 0:
                    rep = x
            if rep is not None:
                self.replace_op(op, rep)
        elif isinstance(op, Sum):
            x, = args
            c = _scalar_const(x)
            if c is not None:
                self.replace_op(op, constant(c * op.reduction_axes.size, op.axes))
        elif isinstance(op, Prod):
            x, = args
            c = _scalar_const(x)
            if c is not None:
                self.replace_op(op, constant(c ** op.reduction_axes.size, op.axes))
        elif isinstance(op, LogOp):
            x, = args
            if isinstance(x, Divide):
                num, denom = self.op_args(x)
                if isinstance(num, ExpOp):
                    exp_x, = self.op_args(num)
                    self.replace_op(op, exp_x - type(op)(denom))
            elif isinstance(x, ExpOp):
                exp_x, = self.op_args(x)
                self.replace_op(op, exp_x)


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


class ReductionLayoutPass(PeepholeGraphPass):
    """Reductions need their reduced axes to form one strided axis.

    When they do not, the operand is first copied into (reduced..., kept...)
    order; this is the layout conversion the reference inserts as a
    DimshuffleOp for the same reason (gpulayout.py:861-979,
    layout_common.py:347-378).
    """

    def visit(self, op, *args):
        from ngraph_hip.op_graph.op_graph import ReductionOp
        if not isinstance(op, ReductionOp) or len(op.reduction_axes) < 2:
            return
        x, = args
        if axes_merge_to_one(x.tensor_description(), op.reduction_axes):
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
