"""Mean, variance and the reciprocal root of rows in one pass over the operand: the graph op the
fusion pass puts in place of ng.mean / ng.variance (op_graph.py:4007-4009, 4252-4266;
layer.py:1242-1257), the pass itself and the kernel that runs `ngh_moments_f32`.
"""
from __future__ import division

import numpy as np

from ngraph_hip.op_graph import op_graph as og
from ngraph_hip.transformers.passes.passes import PeepholeGraphPass
from ngraph_hip.transformers.hipdevice import _td
from ngraph_hip.transformers.hiplowering import HipKernel, _scalar_constant_value, og_unsupported


class MomentsOp(og.TensorOp):
    """mean and variance of x over `reduction_axes` in one read of x.

    Axes = (K,) + kept axes with K of length 3: row 0 holds the mean, row 1 the (biased)
    variance, row 2 -- once `epsilon` is set -- 1/sqrt(variance + epsilon).  Introduced by
    MomentsFusionPass in place of ng.mean + ng.variance (op_graph.py:4007-4009, 4252-4266)
    and of the reciprocal(sqrt(variance + eps)) that batch normalisation takes of it
    (frontends/neon/layer.py:1255); consumers read the rows as slices.
    """

    def __init__(self, x, reduction_axes, **kwargs):
        x = og.as_op(x)
        self.reduction_axes = og.make_axes(reduction_axes)
        self.kept_axes = x.axes - self.reduction_axes
        self.k_axis = og.make_axis(3, name="NGH_MOMENT")
        self.epsilon = None
        super(MomentsOp, self).__init__(args=(x,), axes=og.make_axes([self.k_axis]) + self.kept_axes,
                                        **kwargs)


def moments_layout(td, reduction_axes):
    """(rows, R, row_stride) when `td` is rows x R with contiguous rows over the reduced axes,
    else None."""
    red = [(a.length, td.full_strides[td.axes.index(a)]) for a in reduction_axes if a.length != 1]
    kept = [(a.length, td.full_strides[td.axes.index(a)]) for a in td.axes
            if a not in reduction_axes and a.length != 1]
    red.sort(key=lambda d: -d[1])
    kept.sort(key=lambda d: -d[1])
    for dims in (red, kept):
        for (n0, s0), (n1, s1) in zip(dims[:-1], dims[1:]):
            if s0 != s1 * n1:
                return None
    if not red or red[-1][1] != 1:
        return None
    R = int(np.prod([n for n, _ in red], dtype=np.int64))
    rows = int(np.prod([n for n, _ in kept], dtype=np.int64)) if kept else 1
    row_stride = kept[-1][1] if kept else R
    return rows, R, row_stride


class MomentsFusionPass(PeepholeGraphPass):
    """variance(x) and the mean(x) inside it become one MomentsOp.

    Pattern (after TensorSizeFold): Divide(Sum(Square(Subtract(x, M))), n) with
    M = Divide(Sum(x), n) over the same axes.  Every other Divide(Sum(x), n) over the same x
    and axes is the same mean and is redirected to it as well.  Only applied when x is fp32
    with rows contiguous over the reduced axes (the layout the one-pass kernel handles).
    """

    @staticmethod
    def _strip(op):
        op = op.forwarded
        while isinstance(op, (og.BroadcastOp, og.ReorderAxes)):
            op = op.args[0].forwarded
        return op

    @classmethod
    def _as_mean(cls, op):
        """(x, reduction_axes) when op is Divide(Sum(x), const == size of the reduced axes)."""
        op = cls._strip(op)
        if not isinstance(op, og.Divide):
            return None
        num, den = op.args[0].forwarded, op.args[1].forwarded
        c = _scalar_constant_value(den)
        if not isinstance(num, og.Sum) or c is None or c != float(num.reduction_axes.size):
            return None
        return num.args[0].forwarded, num.reduction_axes

    @staticmethod
    def _same_tensor(a, b):
        ta, tb = _td(a), _td(b)
        return ta.base is tb.base and ta.parameter_key == tb.parameter_key and ta.axes == tb.axes

    def do_pass(self, ops, **kwargs):
        self.moments = []          # (x, reduction axes, mean view, var view)
        self.var_views = {}        # var view -> MomentsOp
        super(MomentsFusionPass, self).do_pass(ops, **kwargs)

    def _visit_rstd(self, op):
        """reciprocal(sqrt(var + c)) of a fused variance becomes row 2 of its MomentsOp."""
        root = self._strip(op.args[0])
        if not isinstance(root, og.SqrtOp):
            return
        add = self._strip(root.args[0])
        if not isinstance(add, og.Add):
            return
        a, b = self._strip(add.args[0]), self._strip(add.args[1])
        for v, c in ((a, b), (b, a)):
            eps = _scalar_constant_value(c)
            mom = self.var_views.get(v)
            if eps is None or mom is None or mom.epsilon not in (None, eps):
                continue
            mom.epsilon = eps
            self.replace_op(op, og.slice_along_axis(mom, mom.k_axis, 2))
            return

    def visit(self, op, *args):
        if isinstance(op, og.ReciprocalOp):
            return self._visit_rstd(op)
        if not isinstance(op, og.Divide):
            return
        outer = self._as_mean(op)
        if outer is None:
            return
        arg, red_axes = outer
        # a mean over x that an earlier match already covers
        for x, axes, mean_view, _ in self.moments:
            if axes.is_equal_set(red_axes) and self._same_tensor(arg, x):
                self.replace_op(op, mean_view)
                return
        if not isinstance(arg, og.SquareOp):
            return
        sub = arg.args[0].forwarded
        if not isinstance(sub, og.Subtract):
            return
        x, m = sub.args[0].forwarded, sub.args[1].forwarded
        inner = self._as_mean(m)
        if inner is None:
            return
        x2, red2 = inner
        if not red2.is_equal_set(red_axes) or not self._same_tensor(x, x2):
            return
        if x.dtype != np.dtype(np.float32):
            return
        if moments_layout(_td(x), red_axes) is None:
            return self._visit_two_level(op, m, x, red_axes)
        mom = MomentsOp(x, red_axes)
        mean_view = og.slice_along_axis(mom, mom.k_axis, 0)
        var_view = og.slice_along_axis(mom, mom.k_axis, 1)
        self.moments.append((x, red_axes, mean_view, var_view))
        self.var_views[var_view] = mom
        self.replace_op(op, var_view)
        self.replace_op(self._strip(m), mean_view)

    def _visit_two_level(self, op, m, x, red_axes):
        """The reduced axes do not form one run of contiguous rows, but some of them do (sum over
        N, H and W of an [N, C, H, W] tensor: rows of H*W elements): one-pass moments of those
        rows, then the rows' statistics are combined over the remaining axes, which is exact
        for rows of equal length:  mean = E[mean_row],  var = E[var_row + (mean_row - mean)^2].
        One read of x instead of two, and no copy of x into (reduced, kept) order."""
        td = _td(x)
        inner = [a for a in red_axes if a.length != 1 and td.full_strides[td.axes.index(a)] == 1]
        if len(inner) != 1:
            return
        # grow the run of rows outwards while the next reduced axis continues it
        run, stride = list(inner), inner[0].length
        grown = True
        while grown:
            grown = False
            for a in red_axes:
                if a not in run and a.length != 1 and td.full_strides[td.axes.index(a)] == stride:
                    run.append(a)
                    stride *= a.length
                    grown = True
        outer = [a for a in red_axes if a not in run]
        R = int(np.prod([a.length for a in run]))
        if not outer or R < 64 or moments_layout(td, og.make_axes(run)) is None:
            return
        mom = MomentsOp(x, og.make_axes(run))
        row_mean = og.slice_along_axis(mom, mom.k_axis, 0)
        row_var = og.slice_along_axis(mom, mom.k_axis, 1)
        n_rows = float(np.prod([a.length for a in outer]))
        mean = og.sum(row_mean, reduction_axes=outer) / n_rows
        var = og.sum(row_var + og.square(row_mean - mean), reduction_axes=outer) / n_rows
        self.moments.append((x, red_axes, mean, var))
        self.replace_op(op, var)
        self.replace_op(self._strip(m), mean)


class MomentsKernel(HipKernel):
    def __init__(self, transformer, op):
        super(MomentsKernel, self).__init__(transformer)
        self.op = op
        self.name = "moments"
        self.x_cache_hint = 0

    def bind_buffers(self):
        t = self.transformer
        x_td = _td(self.op.args[0].forwarded)
        layout = moments_layout(x_td, self.op.reduction_axes)
        if layout is None:
            raise og_unsupported("MomentsOp operand lost its row layout")
        self.rows, self.R, self.row_stride = layout
        self.x = t.get_tensor_description_tensor_view(x_td)
        self.out = t.get_tensor_description_tensor_view(_td(self.op))
        super(MomentsKernel, self).bind_buffers()

    def buffer_uses(self):
        return [(_td(self.op.args[0].forwarded).base, True, False),
                (_td(self.op).base, False, True)]

    def set_cache_hints(self, hint_of):
        self.x_cache_hint = hint_of(_td(self.op.args[0].forwarded).base, True, False)

    def execute(self):
        out, eps = self.out.ptr, self.op.epsilon
        self.transformer.runtime.moments_f32(self.x.ptr, self.rows, self.R, self.row_stride,
                                             out, out + self.rows * 4,
                                             out + self.rows * 8 if eps is not None else None,
                                             eps or 0.0, self.x_cache_hint)

    def describe(self):
        return [["moments_f32"]]
