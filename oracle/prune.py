"""The algebraic rewrites the reference CPU transformer applies before it generates code.
ORACLE ONLY (test infrastructure).

ngraph/transformers/cputransform.py:905-917 registers SimplePrune ahead of code generation, so
the NumPy statements the CPU transformer runs are those of the *rewritten* graph, and some of
the rewrites change floating-point results (log(exp(x)) becomes x, a sum over a constant
becomes one multiplication).  This module restates the rules of SimplePrune
(passes.py:499-628 under ngraph/transformers/passes/) on its own: one function per rule, looked up by
the class name of the op, applied until nothing changes.  It uses the graph front only for
what a rewrite has to touch -- the `forward` pointer of an op and the constructors of the
replacement ops.
"""
import numpy as np

from ngraph_hip.op_graph import op_graph as og


def _args(op):
    return [a.forwarded for a in op.args]


def _filled_with(x):
    """The value of a scalar constant, else None (`x.is_scalar and x.is_constant`)."""
    if x.is_scalar and x.is_constant:
        return float(np.asarray(x.const).reshape(()))
    return None


def _negative(op):                                    # passes.py:512-523
    c = _filled_with(_args(op)[0])
    return None if c is None else og.constant(-c, op.axes)


def _multiply(op):                                    # passes.py:525-552
    x, y = _args(op)
    for fixed, other in ((x, y), (y, x)):
        c = _filled_with(fixed)
        if c is None:
            continue
        # the reference looks at y only when x is no scalar constant
        if c == 0:
            return fixed
        if c == 1:
            return other
        if c == -1:
            return og.negative(other)
        return None
    return None


def _add(op):                                         # passes.py:554-577
    x, y = _args(op)
    if _filled_with(x) is not None:
        return y if _filled_with(x) == 0 else None
    if _filled_with(y) is not None:
        return x if _filled_with(y) == 0 else None
    if type(y).__name__ == "ContiguousOp":
        inner = _args(y)[0]
        if type(inner).__name__ == "BroadcastOp" and _filled_with(_args(inner)[0]) == 0:
            return x
    return None


def _sum(op):                                         # passes.py:579-592
    c = _filled_with(_args(op)[0])
    return None if c is None else og.constant(c * op.reduction_axes.size, op.axes)


def _prod(op):                                        # passes.py:594-608
    c = _filled_with(_args(op)[0])
    return None if c is None else og.constant(c ** op.reduction_axes.size, op.axes)


def _log(op):                                         # passes.py:610-628
    x = _args(op)[0]
    if type(x).__name__ == "Divide":
        num, denom = _args(x)
        if type(num).__name__ == "ExpOp":
            return _args(num)[0] - type(op)(denom)
    elif type(x).__name__ == "ExpOp":
        return _args(x)[0]
    return None


RULES = {"NegativeOp": _negative, "Multiply": _multiply, "Add": _add, "Sum": _sum,
         "Prod": _prod, "LogOp": _log}


def _rule_for(op):
    for cls in type(op).__mro__:
        if cls.__name__ in RULES:
            return RULES[cls.__name__]
    return None


class OraclePrune(object):
    """Graph pass object (`wrapped_do_pass(ops=roots)`): sweeps over the graph in dependency
    order, collecting replacements, and applies them after each sweep, as the reference's
    PeepholeGraphPass does (passes.py:67-84); a replacement takes the axes of the op it
    replaces (passes.py:86-120)."""

    def wrapped_do_pass(self, ops, **kwargs):
        while True:
            found = []
            for op in og.Op.ordered_ops(ops):
                op = op.forwarded
                rule = _rule_for(op)
                rep = rule(op) if rule is not None else None
                if rep is None:
                    continue
                rep = og.as_op(rep)
                if op.is_tensor_op and rep.axes != op.axes:
                    rep = og.axes_with_order(og.broadcast(rep, op.axes), op.axes)
                found.append((op, rep))
            if not found:
                return
            for op, rep in found:
                old, new = op.forwarded, rep.forwarded
                if new is not old:
                    old.forward = new
