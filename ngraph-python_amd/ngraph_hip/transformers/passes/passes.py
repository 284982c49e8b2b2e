"""Graph passes run before lowering: the part that ngraph/transformers/passes/passes.py
provides in the reference -- the pass driver (passes.py:35-120), `replace_op` with axes
repair, and the `SimplePrune` algebra (passes.py:499-628) that changes which ops reach the
kernels (x*1, x*0, x*-1, x+0, constant sum/prod, log(exp x), -const).  The passes that are
this backend's own live in hippasses.py.
"""
from __future__ import division
import numpy as np

from ngraph_hip.op_graph.op_graph import (
    Op, NegativeOp, Multiply, Add, Sum, Prod, LogOp, ExpOp, Divide, ContiguousOp,
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
