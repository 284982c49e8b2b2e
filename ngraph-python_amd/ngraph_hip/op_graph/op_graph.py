"""Op-graph front for the elementwise / reduction path.

A compact counterpart of ngraph/op_graph/op_graph.py: the same constructor
names, axes rules and ordering semantics for the ops the fused kernels cover,
so graphs written for the reference build unchanged.  What is mirrored:

* tensor kinds placeholder / variable / persistent_tensor / temporary /
  constant (op_graph.py:2297-2564); reads of state go through TensorValueOp
  (op_graph.py:787-806, 1593-1617);
* binary elementwise axes `x.axes + (y.axes - x.axes)` unless y already has
  them all, operands broadcast and reordered as views (op_graph.py:3159-3180);
* reductions with reduction_axes / out_axes (op_graph.py:3853-3932), mean,
  variance (two-pass), tensor_size (op_graph.py:4007-4046, 4252-4266);
* views that never run on the device: broadcast, axes_with_order, flatten,
  unflatten, tensor_slice, cast_axes, expand_dims, Transpose
  (op_graph.py:1650-2295);
* assign / sequential / computation with state read-write ordering
  (op_graph.py:821-912, 961-1033, 1494-1590);
* execution order = topological sort over args and control deps following
  `forwarded` (op_graph.py:244-292).

Autodiff, dot / convolution / pooling / lookup ops are outside this path.
"""
from __future__ import division
from collections import OrderedDict, defaultdict
import builtins
import numbers

import numpy as np

from ngraph_hip.op_graph.axes import (Axes, Axis, FlattenedAxis, TensorDescription, make_axes,
                                      make_axis, default_dtype, default_int_dtype, slice_axis)


class OrderedSet(object):
    """Insertion-ordered set (the reference uses the `orderedset` package)."""

    def __init__(self, items=()):
        self._d = OrderedDict()
        self.update(items)

    def add(self, x):
        self._d[x] = None

    def update(self, items):
        for x in items:
            self._d[x] = None

    def discard(self, x):
        self._d.pop(x, None)

    def pop(self):
        return self._d.popitem()[0]

    def __contains__(self, x):
        return x in self._d

    def __iter__(self):
        return iter(self._d)

    def __len__(self):
        return len(self._d)

    def __or__(self, other):
        out = OrderedSet(self)
        out.update(other)
        return out

    def __bool__(self):
        return bool(self._d)

    __nonzero__ = __bool__


_name_counters = defaultdict(int)


def _auto_name(cls):
    n = _name_counters[cls.__name__]
    _name_counters[cls.__name__] += 1
    return "%s_%d" % (cls.__name__, n)


class Op(object):
    """Any node of the graph."""

    def __init__(self, args=(), metadata=None, const=None, constant=False, name=None, **kwargs):
        self._args = None
        self._control_deps = OrderedSet()
        self._forward = None
        self.metadata = dict(metadata or {})
        self._const = const
        self._is_constant = constant
        self.name = name if name is not None else _auto_name(type(self))
        self.args = args

    # -- structure ---------------------------------------------------------------
    @property
    def args(self):
        return self._args

    @args.setter
    def args(self, args):
        self._args = tuple(as_op(a) for a in args)

    @property
    def control_deps(self):
        return self._control_deps

    def add_control_dep(self, dep):
        dep = dep.forwarded
        if dep is not self.forwarded:
            self._control_deps.add(dep)

    @property
    def all_deps(self):
        return OrderedSet(a.forwarded for a in self.args) | OrderedSet(d.forwarded for d in self._control_deps)

    @property
    def forward(self):
        return self._forward

    @forward.setter
    def forward(self, value):
        self._forward = value

    @property
    def forwarded(self):
        """The op to use instead of this one after graph rewrites (op_graph.py:554-578)."""
        result = self
        while result._forward is not None:
            result = result._forward
        return result

    def named(self, name):
        self.name = name
        return self

    @property
    def safe_name(self):
        return self.name.replace(".", "_").replace("-", "_")

    # -- classification ------------------------------------------------------------
    @property
    def is_tensor_op(self):
        return False

    @property
    def is_device_op(self):
        """True when the op computes on the device (views and sequencing ops do not)."""
        return True

    @property
    def is_state_op(self):
        return False

    @property
    def is_sequencing_op(self):
        return False

    @property
    def has_side_effects(self):
        return False

    @property
    def is_constant(self):
        return self._is_constant

    @property
    def const(self):
        return self._const

    @property
    def is_scalar(self):
        return False

    @property
    def tensor(self):
        return self

    # -- state tracking ----------------------------------------------------------------
    @property
    def states_read(self):
        out = OrderedSet()
        for a in self.args:
            out.update(a.forwarded.states_read)
        return out

    @property
    def states_written(self):
        out = OrderedSet()
        for a in self.args:
            out.update(a.forwarded.states_written)
        return out

    def __repr__(self):
        return "<%s(%s)>" % (type(self).__name__, self.name)

    # -- traversal -------------------------------------------------------------------
    @staticmethod
    def ordered_ops(roots):
        """Topological order over args and control deps (op_graph.py:244-292)."""
        ordered, available, counts = [], OrderedSet(), dict()
        parents, ready = defaultdict(OrderedSet), OrderedSet()
        available.update(root.forwarded for root in roots)
        while available:
            node = available.pop()
            if node in counts or node in ready:
                continue
            children = node.all_deps
            if children:
                counts[node] = len(children)
                for child in children:
                    parents[child].add(node)
                available.update(children)
            else:
                ready.add(node)
        while ready:
            node = ready.pop()
            ordered.append(node)
            for p in parents.get(node, []):
                count = counts[p] - 1
                if count == 0:
                    ready.add(p)
                    del counts[p]
                else:
                    counts[p] = count
        if len(counts) > 0:
            raise ValueError("Graph not a DAG")
        return ordered


def as_op(x):
    """An Op for x: state tensors are read through TensorValueOp, scalars become constants."""
    if isinstance(x, AssignableTensorOp):
        return TensorValueOp(x)
    if isinstance(x, Op):
        return x
    return TensorValueOp(constant(x))


def as_ops(xs):
    return tuple(as_op(x) for x in xs)


# =============================================================================== control
class AssignOp(Op):
    """tensor[...] = val (op_graph.py:821-861)."""

    def __init__(self, tensor, val, **kwargs):
        if not isinstance(val, Op):
            val = as_op(val)
            if len(val.axes) == len(tensor.axes):
                val = cast_axes(val, tensor.axes)
        if len(val.axes - tensor.axes) > 0:
            raise ValueError("tensor(LHS) has axes %s. val(RHS) has axes %s. val's axes should be "
                             "subset of tensor's axes" % (val.axes, tensor.axes))
        val = broadcast(val, tensor.axes)
        super(AssignOp, self).__init__(args=(tensor, val), **kwargs)

    @property
    def states_written(self):
        return self.args[0].forwarded.states_read

    @property
    def states_read(self):
        return self.args[1].forwarded.states_read

    @property
    def has_side_effects(self):
        return True


def assign(lvalue, rvalue):
    return AssignOp(lvalue, rvalue)


class ControlBlockOp(Op):
    @property
    def is_device_op(self):
        return False


class ParallelOp(ControlBlockOp):
    """Compute every op in any order compatible with existing dependencies."""

    def __init__(self, all, **kwargs):
        super(ParallelOp, self).__init__(**kwargs)
        for op in all:
            self.add_control_dep(as_op(op))


def doall(all):
    return ParallelOp(all)


class ComputationOp(ParallelOp):
    """A callable unit: what to return and which placeholders are arguments (op_graph.py:961-1018)."""

    def __init__(self, returns, *args, **kwargs):
        super(ComputationOp, self).__init__(all=(), **kwargs)

        def wrap_op(op):
            if isinstance(op, (list, tuple, set)):
                raise ValueError("nested return containers are not supported")
            return as_op(op)

        self.returns_kind = None
        if isinstance(returns, (list, tuple)):
            self.returns = [wrap_op(r) for r in returns]
            self.returns_kind = "sequence"
            self.values = list(self.returns)
        elif isinstance(returns, set):
            self.returns_map = OrderedDict((r, wrap_op(r)) for r in returns)
            self.returns = self.returns_map
            self.returns_kind = "set"
            self.values = list(self.returns_map.values())
        elif isinstance(returns, Op) or returns is not None:
            self.returns = wrap_op(returns)
            self.returns_kind = "op"
            self.values = [self.returns]
        else:
            self.returns = None
            self.returns_kind = "none"
            self.values = []
        for v in self.values:
            self.add_control_dep(v)

        self.parameters = []
        for arg in args:
            if isinstance(arg, TensorValueOp):
                arg = arg.value_tensor
            if not (isinstance(arg, AssignableTensorOp) and arg.is_input):
                raise ValueError("The arguments to a computation must all be Ops with their "
                                 "is_input attribute set (placeholders); got {}".format(arg))
            self.parameters.append(arg)

        # every placeholder the values depend on has to be passed
        used = OrderedSet()
        for op in Op.ordered_ops(self.values):
            used.update(s for s in op.states_read if s.is_placeholder)
        missing = [op for op in used if op not in self.parameters]
        if missing:
            raise ValueError("All used placeholders must be supplied to a computation. "
                             "Missing: {}".format(missing))


def computation(returns, *args):
    return ComputationOp(returns, *args)


class Fill(Op):
    """Fill a tensor with a scalar (op_graph.py:1036-1077)."""

    def __init__(self, tensor, scalar, **kwargs):
        super(Fill, self).__init__(args=(tensor,), **kwargs)
        if isinstance(scalar, TensorOp):
            if scalar.is_constant:
                scalar = scalar.const
            else:
                raise ValueError("{} is not a scalar constant".format(scalar))
        if not isinstance(scalar, numbers.Real) and not np.isscalar(scalar):
            raise ValueError("{} is not a scalar".format(scalar))
        self.scalar = scalar

    @property
    def states_written(self):
        return self.args[0].forwarded.states_read

    @property
    def states_read(self):
        return OrderedSet()

    @property
    def has_side_effects(self):
        return True


def fill(x, scalar):
    return Fill(x, scalar)


# =============================================================================== tensors
class TensorOp(Op):
    """An op that has a tensor value (op_graph.py:1080-1388)."""

    def __init__(self, dtype=None, axes=None, scale=None, is_value_op=False, **kwargs):
        super(TensorOp, self).__init__(**kwargs)
        self.dtype = default_dtype(dtype)
        self._axes = make_axes(axes) if axes is not None else None
        self.scale = scale
        self._td = None

    @property
    def is_tensor_op(self):
        return True

    @property
    def axes(self):
        if self._axes is not None:
            return self._axes
        raise NotImplementedError

    @axes.setter
    def axes(self, value):
        self._axes = make_axes(value)

    @property
    def shape(self):
        return self.axes

    @property
    def tensor(self):
        return self

    @property
    def value_tensor(self):
        return self

    @property
    def effective_tensor_op(self):
        return self

    @property
    def is_scalar(self):
        return 0 == len(self.axes)

    @property
    def has_axes(self):
        return self._axes is not None

    def tensor_description(self):
        """The buffer this op writes: one base description per device op."""
        if self._td is None or self._td.dtype != self.dtype or self._td.axes != self.axes:
            self._td = TensorDescription(self.axes, dtype=self.dtype, name=self.name, op=self,
                                         is_persistent=self.is_persistent, is_input=self.is_input,
                                         is_placeholder=self.is_placeholder)
        return self._td

    def invalidate_tensor_description(self):
        self._td = None

    @property
    def is_persistent(self):
        return False

    @property
    def is_input(self):
        return False

    @property
    def is_placeholder(self):
        return False

    @property
    def is_trainable(self):
        return False

    def mean(self, reduction_axes=None, out_axes=None):
        return mean(self, reduction_axes=reduction_axes, out_axes=out_axes)

    # -- operators (op_graph.py:1185-1256) ---------------------------------------------
    def __neg__(self):
        return negative(self)

    def __pos__(self):
        return self

    def __abs__(self):
        return absolute(self)

    def __add__(self, val):
        return add(self, val)

    def __radd__(self, val):
        return add(val, self)

    def __sub__(self, val):
        return subtract(self, val)

    def __rsub__(self, val):
        return subtract(val, self)

    def __mul__(self, val):
        return multiply(self, val)

    def __rmul__(self, val):
        return multiply(val, self)

    def __truediv__(self, val):
        return divide(self, val)

    def __rtruediv__(self, val):
        return divide(val, self)

    __div__ = __truediv__
    __rdiv__ = __rtruediv__

    def __floordiv__(self, val):
        return floordivide(self, val)

    def __rfloordiv__(self, val):
        return floordivide(val, self)

    def __mod__(self, val):
        return mod(self, val)

    def __pow__(self, val):
        return power(self, val)

    def __rpow__(self, val):
        return power(val, self)

    def __lt__(self, val):
        return less(self, val)

    def __gt__(self, val):
        return greater(self, val)

    def __le__(self, val):
        return less_equal(self, val)

    def __ge__(self, val):
        return greater_equal(self, val)

    # equality stays identity so ops can be dict keys; use ng.equal for the graph op
    def __hash__(self):
        return id(self)

    def __axes__(self):
        return self.axes

    @property
    def T(self):
        return Transpose(self)

    def __getitem__(self, item):
        if isinstance(item, slice) and len(self.axes) > 1:
            item = (item,)
        item += tuple(slice(None) for _ in range(len(self.axes) - len(item)))
        return tensor_slice(self, item)


class ValueOp(TensorOp, ControlBlockOp):
    """An op whose value is another op's (op_graph.py:1390-1492)."""

    def __init__(self, tensor=None, **kwargs):
        super(ValueOp, self).__init__(args=(), is_value_op=True, **kwargs)
        self._tensor = tensor

    def tensor_description(self):
        return self.tensor.tensor_description()

    @property
    def is_device_op(self):
        return False

    @property
    def tensor(self):
        if self._tensor is not None:
            return self._tensor.forwarded.tensor.forwarded
        return None

    @property
    def value_tensor(self):
        if self._tensor is not None:
            return self._tensor.forwarded
        return None

    @value_tensor.setter
    def value_tensor(self, tensor):
        self._tensor = tensor

    @property
    def all_deps(self):
        base = super(ValueOp, self).all_deps
        vt = self.value_tensor
        if vt is not None and (vt.is_device_op or isinstance(vt, (IndexOp, ValueOp))):
            return base | OrderedSet([vt])
        return base

    @property
    def is_tensor_op(self):
        return self.tensor.is_tensor_op

    @property
    def axes(self):
        return self.tensor.axes

    @property
    def dtype(self):
        if self._tensor is not None and self.tensor.is_tensor_op:
            return self.tensor.dtype
        return default_dtype(None)

    @dtype.setter
    def dtype(self, dtype):
        if getattr(self, "_tensor", None) is not None:
            self.tensor.dtype = default_dtype(dtype)

    @property
    def is_constant(self):
        return self.tensor.is_constant

    @property
    def const(self):
        return self.tensor.const

    @property
    def is_scalar(self):
        return self.tensor.is_scalar

    @property
    def states_read(self):
        return self.value_tensor.states_read

    @property
    def states_written(self):
        return self.value_tensor.states_written

    @property
    def effective_tensor_op(self):
        tensor = self._tensor
        if tensor.is_state_op:
            return self.forwarded
        return tensor.effective_tensor_op


class SequentialOp(ValueOp):
    """Run ops once, in order; value = the last op (op_graph.py:1494-1572)."""

    def __init__(self, ops=None, **kwargs):
        super(SequentialOp, self).__init__(**kwargs)
        self.value_tensor = None
        self._ops = None
        if ops is not None:
            self.ops = ops

    @property
    def ops(self):
        return self._ops

    @ops.setter
    def ops(self, ops):
        self._ops = list(as_op(op).forwarded for op in ops)
        for op in self._ops:
            self.add_control_dep(op)
        self.value_tensor = self._ops[-1]
        done_ops = set()
        writers = defaultdict(OrderedSet)
        readers = defaultdict(OrderedSet)
        for op_top in self._ops:
            ordered = Op.ordered_ops([op_top])
            for op in ordered:
                if op in done_ops:
                    continue
                for state in op.states_read:
                    for write_op in writers[state]:
                        op.add_control_dep(write_op)
                for state in op.states_written:
                    for read_op in readers[state]:
                        op.add_control_dep(read_op)
                    for write_op in writers[state]:
                        op.add_control_dep(write_op)
            for op in ordered:
                if op in done_ops:
                    continue
                for state in op.states_written:
                    writers[state].add(op_top)
                for state in op.states_read:
                    readers[state].add(op_top)
            done_ops.update(ordered)

    @property
    def is_sequencing_op(self):
        return True

    @property
    def is_tensor_op(self):
        vt = self.value_tensor
        return vt is not None and vt.is_tensor_op


def sequential(ops=None):
    return SequentialOp(ops)


class TensorValueOp(ValueOp):
    """A read of an AssignableTensorOp (op_graph.py:1593-1617)."""

    def __init__(self, tensor, **kwargs):
        super(TensorValueOp, self).__init__(tensor=tensor, **kwargs)

    @property
    def states_read(self):
        return OrderedSet([self.tensor])

    @property
    def states_written(self):
        return OrderedSet()

    @property
    def all_deps(self):
        return OrderedSet(d.forwarded for d in self._control_deps)

    @property
    def effective_tensor_op(self):
        return self.forwarded


# =============================================================================== views
class IndexOp(TensorOp):
    """An op that only re-describes its argument's storage (op_graph.py:1650-1721)."""

    def __init__(self, x, **kwargs):
        super(IndexOp, self).__init__(args=(x,), dtype=x.dtype, **kwargs)

    @property
    def is_device_op(self):
        return False

    @property
    def dtype(self):
        return self.args[0].forwarded.dtype if self._args else self._dtype

    @dtype.setter
    def dtype(self, value):
        self._dtype = default_dtype(value)

    def transform_tensor_description(self, tensor_description):
        raise NotImplementedError

    def tensor_description(self):
        return self.transform_tensor_description(self.args[0].forwarded.tensor_description())

    @property
    def is_scalar(self):
        return self.args[0].forwarded.is_scalar

    @property
    def is_constant(self):
        return self.args[0].forwarded.is_constant

    @property
    def const(self):
        return self.args[0].forwarded.const

    @property
    def is_persistent(self):
        return self.args[0].forwarded.is_persistent


class Transpose(IndexOp):
    def __init__(self, x, **kwargs):
        super(Transpose, self).__init__(x, axes=make_axes(tuple(reversed(x.axes))), **kwargs)

    def transform_tensor_description(self, td):
        return td.transpose()


class AxesCastOp(IndexOp):
    def __init__(self, x, axes, **kwargs):
        axes = make_axes(axes)
        if axes.lengths != x.axes.lengths:
            raise ValueError("casting axes {} must have the same length as original axes {}"
                             .format(axes, x.axes))
        super(AxesCastOp, self).__init__(x, axes=axes, **kwargs)

    def transform_tensor_description(self, td):
        return td.cast(self.axes)


def cast_axes(tensor, axes):
    axes = make_axes(axes)
    if tensor.axes.lengths != axes.lengths:
        raise ValueError("casting axes {} must have the same length as original axes {}"
                         .format(axes, tensor.axes))
    if len(axes.lengths) == 0:
        return tensor
    return AxesCastOp(tensor, axes)


def cast_role(tensor, axes):
    return cast_axes(tensor, axes)


class ExpandDims(IndexOp):
    def __init__(self, x, axis, dim, **kwargs):
        axes = list(x.axes)
        axes.insert(dim, axis)
        self.axis, self.dim = axis, dim
        super(ExpandDims, self).__init__(x, axes=make_axes(axes), **kwargs)

    def transform_tensor_description(self, td):
        return td.broadcast(self.axes)


def expand_dims(x, axis, dim):
    if axis in x.axes:
        return x
    return ExpandDims(x, axis, dim)


class BroadcastOp(IndexOp):
    def __init__(self, x, axes, **kwargs):
        Axes.assert_valid_broadcast(x.axes, axes)
        super(BroadcastOp, self).__init__(x, axes=axes, **kwargs)

    def transform_tensor_description(self, td):
        return td.broadcast(self.axes)


def broadcast(x, axes):
    axes = make_axes(axes)
    x = as_op(x)
    if x.axes == axes:
        return x
    return BroadcastOp(x, axes)


def axes_with_order(x, axes):
    axes = make_axes(axes)
    if x.axes == axes:
        return x
    return ReorderAxes(x, axes)


class ReorderAxes(IndexOp):
    def __init__(self, x, axes, **kwargs):
        if not x.axes.is_equal_set(axes):
            raise ValueError("The input and output axes must have the same elements.")
        super(ReorderAxes, self).__init__(x, axes=axes, **kwargs)

    def transform_tensor_description(self, td):
        return td.reorder(self.axes)


def tensor_slice(x, slices, axes=None):
    return TensorSliceOp(x, slices, axes)


class TensorSliceOp(IndexOp):
    def __init__(self, x, slices, axes=None, **kwargs):
        slices = tuple(slices)
        if len(slices) != len(x.axes):
            raise ValueError("There should be one slice in slices for each dimension in input "
                             "tensor.  Input tensor had {} dimensions, but slices has length {}."
                             .format(len(x.axes), len(slices)))
        for s in slices:
            if isinstance(s, slice) and s.step not in (None, 1):
                raise ValueError("slices with a step need a copy and are not supported as views")
        if axes is None:
            axes = []
            for axis, s in zip(x.axes, slices):
                if isinstance(s, slice):
                    axes.append(slice_axis(axis, s))
            axes = make_axes(axes)
        self.slices = slices
        super(TensorSliceOp, self).__init__(x, axes=axes, **kwargs)

    def transform_tensor_description(self, td):
        return td.slice(self.slices, self.axes)


def slice_along_axis(x, axis, idx):
    pos = x.axes.index(axis)
    ss = tuple(idx if i == pos else slice(None) for i in range(len(x.axes)))
    axes = x.axes[:pos] + x.axes[pos + 1:]
    return tensor_slice(x, ss, axes=axes)


class Flatten(IndexOp):
    def __init__(self, x, axes, **kwargs):
        x = ContiguousOp(axes_with_order(x, x.axes)) if not isinstance(x, ContiguousOp) and \
            not _flattenable(x, axes) else x
        super(Flatten, self).__init__(x, axes=axes, **kwargs)

    def transform_tensor_description(self, td):
        return td.flatten(self.axes)


def _flattenable(x, axes):
    try:
        return x.tensor_description().can_flatten(axes)
    except Exception:
        return False


def flatten(x, axes=None, **kwargs):
    if axes is None:
        if len(x.axes) == 1:
            return x
        axes = make_axes((FlattenedAxis(x.axes),))
    axes = make_axes(axes)
    if x.axes == axes:
        return x
    return Flatten(x, axes, **kwargs)


def flatten_at(x, idx):
    if idx == 0 or idx == len(x.axes):
        return flatten(x)
    return flatten(x, make_axes((make_axes(x.axes[:idx]).flatten(), make_axes(x.axes[idx:]).flatten())))


class Unflatten(IndexOp):
    def __init__(self, x, axes=None, **kwargs):
        if axes is None:
            axes = []
            for axis in x.axes:
                axes.extend(axis.axes if axis.is_flattened else [axis])
        axes = make_axes(axes)
        super(Unflatten, self).__init__(x, axes=axes, **kwargs)

    def transform_tensor_description(self, td):
        return td.unflatten(self.axes)


def unflatten(x, axes=None, **kwargs):
    if not any(a.is_flattened for a in x.axes):
        return x
    return Unflatten(x, axes=axes, **kwargs)


class ContiguousOp(TensorOp):
    """Materialise a view as a C-contiguous tensor (op_graph.py:3670-3686); a device copy."""

    def __init__(self, x, **kwargs):
        super(ContiguousOp, self).__init__(args=(x,), axes=x.axes, dtype=x.dtype, **kwargs)

    @property
    def old_axes(self):
        return self.args[0].forwarded.axes


# =============================================================================== state
class AssignableTensorOp(TensorOp):
    """A tensor with storage of its own that can be written (op_graph.py:2297-2424)."""

    def __init__(self, initial_value=None, is_constant=False, is_input=False, is_persistent=False,
                 is_trainable=False, is_placeholder=False, const=None, scope=None, **kwargs):
        super(AssignableTensorOp, self).__init__(const=const, constant=is_constant, **kwargs)
        self._is_input = is_input
        self._is_persistent = is_persistent
        self._is_trainable = is_trainable
        self._is_placeholder = is_placeholder
        self.initial_value = None
        if initial_value is not None:
            if callable(initial_value):
                initial_value = initial_value(self.axes)
            if isinstance(initial_value, TensorOp):
                # a constant op stands for its value (op_graph.py:2338-2344)
                tensor = initial_value.forwarded.tensor
                if not getattr(tensor, "is_constant", False) or tensor.const is None:
                    raise ValueError("initial_value must be convertible to a NumPy tensor")
                initial_value = tensor.const
            # a private copy: later changes to the caller's array must not reach the graph
            self.initial_value = np.array(initial_value, dtype=np.float64 if not isinstance(
                self.dtype, np.dtype) else self.dtype, copy=True)

    @property
    def is_device_op(self):
        return False

    @property
    def is_state_op(self):
        return True

    @property
    def is_persistent(self):
        return self._is_persistent

    @property
    def is_input(self):
        return self._is_input

    @property
    def is_placeholder(self):
        return self._is_placeholder

    @property
    def is_trainable(self):
        return self._is_trainable

    @property
    def states_read(self):
        return OrderedSet([self])

    @property
    def states_written(self):
        return OrderedSet()

    @property
    def all_deps(self):
        return OrderedSet()


def value_of(tensor):
    if tensor.is_constant:
        return tensor
    temp = temporary(axes=tensor.axes, dtype=tensor.dtype).named("value_of_" + tensor.name)
    return sequential([AssignOp(temp, tensor), temp])


def constant(const, axes=None, dtype=None, **kwargs):
    """A constant tensor; a scalar given axes is broadcast to them (op_graph.py:2445-2477)."""
    nptensor = np.asarray(const, dtype=dtype if isinstance(dtype, np.dtype) or dtype is None else None)
    if axes and len(axes) == len(nptensor.shape):
        nptensor_axes = axes
    else:
        nptensor_axes = make_axes([make_axis(l) for l in nptensor.shape])
    graph_label_type = "<Const({})>".format(const)
    val = AssignableTensorOp(axes=nptensor_axes, is_constant=True, is_persistent=True,
                             is_trainable=False, initial_value=nptensor, const=nptensor,
                             dtype=dtype, **kwargs)
    val.graph_label_type = graph_label_type
    if axes and len(axes) > 0 and val.is_scalar:
        val = broadcast(val, axes)
    return val


def placeholder(axes, dtype=None, initial_value=None, **kwargs):
    return AssignableTensorOp(axes=make_axes(axes), is_constant=False, is_input=True,
                              is_persistent=True, is_trainable=False, is_placeholder=True,
                              initial_value=initial_value, dtype=dtype, **kwargs)


def temporary(axes, dtype=None, **kwargs):
    # op_graph.py:2501-2519: storage a computation may reuse; not an input
    return AssignableTensorOp(axes=make_axes(axes), is_constant=False, is_input=False,
                              is_persistent=False, is_trainable=False, dtype=dtype, **kwargs)


def persistent_tensor(axes, dtype=None, initial_value=None, **kwargs):
    return AssignableTensorOp(axes=make_axes(axes), is_constant=False, is_input=True,
                              is_persistent=True, is_trainable=False,
                              initial_value=initial_value, dtype=dtype, **kwargs)


def variable(axes, dtype=None, initial_value=None, scope=None, **kwargs):
    return AssignableTensorOp(axes=make_axes(axes), is_constant=False, is_input=True,
                              is_persistent=True, is_trainable=True,
                              initial_value=initial_value, dtype=dtype, scope=scope, **kwargs)


# =============================================================================== elementwise
class ElementWiseOp(TensorOp):
    pass


class UnaryElementWiseOp(ElementWiseOp):
    def __init__(self, x, **kwargs):
        x = as_op(x)
        super(UnaryElementWiseOp, self).__init__(args=(x,), axes=x.axes, **kwargs)


def _unary(name, doc):
    cls = type(name, (UnaryElementWiseOp,), {"__doc__": doc})
    return cls


NegativeOp = _unary("NegativeOp", "-x (op_graph.py:2903-2910)")
AbsoluteOp = _unary("AbsoluteOp", "|x| (op_graph.py:2925-2932)")
SinOp = _unary("SinOp", "sin x")
CosOp = _unary("CosOp", "cos x")
TanhOp = _unary("TanhOp", "tanh x")
ExpOp = _unary("ExpOp", "exp x")
LogOp = _unary("LogOp", "log x")
ReciprocalOp = _unary("ReciprocalOp", "1 / x")
SignOp = _unary("SignOp", "sign x")
SquareOp = _unary("SquareOp", "x * x")
SqrtOp = _unary("SqrtOp", "sqrt x")
SigmoidAtomicOp = _unary("SigmoidAtomicOp", "1 / (1 + exp(-x)) as one op (op_graph.py:4205-4223)")


def negative(x):
    return NegativeOp(x)


def absolute(x):
    return AbsoluteOp(x)


def sin(x):
    return SinOp(x)


def cos(x):
    return CosOp(x)


def tanh(x):
    return TanhOp(x)


def exp(x):
    return ExpOp(x)


def log(x):
    return LogOp(x)


safelog_cutoff = 50.0


def safelog(x, limit=-safelog_cutoff):
    """log(x) cut off below at `limit`: maximum(log(x + exp(limit)), limit)
    (op_graph.py:3070-3072).  safelog(0) is `limit`; a negative x gives NaN, as log does."""
    offset = np.exp(limit)
    return maximum(log(x + offset), limit)


def reciprocal(x):
    return ReciprocalOp(x)


def sign(x):
    return SignOp(x)


def square(x):
    return SquareOp(x)


def sqrt(x):
    return SqrtOp(x)


class BinaryElementWiseOp(ElementWiseOp):
    def __init__(self, x, y, **kwargs):
        x, y = as_ops((x, y))
        x_axes_bcast = x.axes + (y.axes - x.axes)
        y_axes_bcast = y.axes + (x.axes - y.axes)
        if y_axes_bcast == y.axes:
            axes = y_axes_bcast
        else:
            axes = x_axes_bcast
        x = axes_with_order(broadcast(x, x_axes_bcast), axes)
        y = axes_with_order(broadcast(y, y_axes_bcast), axes)
        super(BinaryElementWiseOp, self).__init__(args=(x, y), axes=axes, **kwargs)


class CommutativeBinaryElementWiseOp(BinaryElementWiseOp):
    @property
    def is_commutative(self):
        return True


def _binary(name, commutative=False):
    base = CommutativeBinaryElementWiseOp if commutative else BinaryElementWiseOp
    return type(name, (base,), {})


Add = _binary("Add", True)
Subtract = _binary("Subtract")
Multiply = _binary("Multiply", True)
Divide = _binary("Divide")
FloorDivide = _binary("FloorDivide")
Mod = _binary("Mod")
Maximum = _binary("Maximum", True)
Minimum = _binary("Minimum", True)
Power = _binary("Power")
Equal = _binary("Equal", True)
NotEqual = _binary("NotEqual", True)
Greater = _binary("Greater")
Less = _binary("Less")
GreaterEqual = _binary("GreaterEqual")
LessEqual = _binary("LessEqual")


def add(x, y, dtype=None):
    return Add(x, y, dtype=dtype)


def subtract(x, y, dtype=None):
    return Subtract(x, y, dtype=dtype)


def multiply(x, y, dtype=None):
    return Multiply(x, y, dtype=dtype)


def divide(x, y, dtype=None):
    return Divide(x, y, dtype=dtype)


def floordivide(x, y, dtype=None):
    return FloorDivide(x, y, dtype=dtype)


def mod(x, y, dtype=None):
    return Mod(x, y, dtype=dtype)


def maximum(x, y, dtype=None):
    return Maximum(x, y, dtype=dtype)


def minimum(x, y, dtype=None):
    return Minimum(x, y, dtype=dtype)


def power(x, y, dtype=None):
    return Power(x, y, dtype=dtype)


def equal(x, y, dtype=None):
    return Equal(x, y, dtype=dtype)


def not_equal(x, y, dtype=None):
    return NotEqual(x, y, dtype=dtype)


def greater(x, y, dtype=None):
    return Greater(x, y, dtype=dtype)


def less(x, y, dtype=None):
    return Less(x, y, dtype=dtype)


def greater_equal(x, y, dtype=None):
    return GreaterEqual(x, y, dtype=dtype)


def less_equal(x, y, dtype=None):
    return LessEqual(x, y, dtype=dtype)


# =============================================================================== reductions
class ReductionOp(TensorOp):
    def __init__(self, x, reduction_axes=None, out_axes=None, dtype=None, **kwargs):
        x = as_op(x)
        reduction_axes, out_axes = compute_reduction_axes(x, reduction_axes, out_axes)
        self.reduction_axes = reduction_axes
        super(ReductionOp, self).__init__(args=(x,), axes=out_axes, dtype=dtype, **kwargs)


def compute_reduction_axes(x, reduction_axes, out_axes):
    # op_graph.py:3871-3900
    if reduction_axes is None and out_axes is None:
        rec = x.axes.recurrent_axis()
        reduction_axes = x.axes.sample_axes() - (make_axes(rec) if rec is not None else make_axes(()))
        out_axes = x.axes - reduction_axes
    elif reduction_axes is None:
        out_axes = make_axes(out_axes)
        reduction_axes = x.axes - out_axes
    elif out_axes is None:
        reduction_axes = make_axes(reduction_axes)
        out_axes = x.axes - reduction_axes
    else:
        out_axes = make_axes(out_axes)
        reduction_axes = make_axes(reduction_axes)
    if not reduction_axes & out_axes == make_axes(()):
        raise ValueError("reduction_axes {} and out_axes {} must not overlap"
                         .format(reduction_axes, out_axes))
    if not (reduction_axes | out_axes).is_equal_set(x.axes):
        raise ValueError("union of reduction_axes {} and out_axes {} must be x.axes {}"
                         .format(reduction_axes, out_axes, x.axes))
    out_axes_index = [x.axes.index(axis) for axis in out_axes]
    if sorted(out_axes_index) != out_axes_index:
        raise ValueError("out_axes {} must has same order as x.axes {}".format(out_axes, x.axes))
    return reduction_axes, out_axes


def create_reduction_op(name, func_name=None):
    RedClass = type(name, (ReductionOp,), {})

    def func(*args, **kwargs):
        if "out_axes" in kwargs and kwargs["out_axes"] is not None:
            x = as_op(args[0])
            out_axes = make_axes(kwargs["out_axes"])
            out_axes_index = [x.axes.index(axis) for axis in out_axes]
            sorted_index = sorted(out_axes_index)
            if sorted_index != out_axes_index:
                kwargs["out_axes"] = [x.axes[i] for i in sorted_index]
                return axes_with_order(RedClass(*args, **kwargs), out_axes)
        return RedClass(*args, **kwargs)

    func.__name__ = func_name
    return RedClass, func


Max, max = create_reduction_op("Max", "max")
Min, min = create_reduction_op("Min", "min")
Sum, sum = create_reduction_op("Sum", "sum")
Prod, prod = create_reduction_op("Prod", "prod")
Argmax, _ = create_reduction_op("Argmax", "argmax")
Argmin, _ = create_reduction_op("Argmin", "argmin")


def argmax(x, dtype=None, **kwargs):
    return Argmax(x, dtype=default_int_dtype(dtype), **kwargs)


def argmin(x, dtype=None, **kwargs):
    return Argmin(x, dtype=default_int_dtype(dtype), **kwargs)


def variance(x, out_axes=None, reduction_axes=None):
    # two-pass, op_graph.py:4007-4009
    return mean(square(x - mean(x, out_axes=out_axes, reduction_axes=reduction_axes)),
                out_axes=out_axes, reduction_axes=reduction_axes)


class TensorSizeOp(TensorOp):
    """A scalar holding the number of elements reduced (op_graph.py:4012-4031)."""

    def __init__(self, x, reduction_axes=None, out_axes=None, **kwargs):
        x = as_op(x)
        if reduction_axes is None and out_axes is None:
            reduction_axes = x.axes.sample_axes()
        elif reduction_axes is None:
            reduction_axes = x.axes - make_axes(out_axes)
        self.reduction_axes = make_axes(reduction_axes)
        super(TensorSizeOp, self).__init__(args=(x,), axes=(), **kwargs)


def tensor_size(x, reduction_axes=None, out_axes=None):
    return TensorSizeOp(x, reduction_axes=reduction_axes, out_axes=out_axes)


def batch_size(x):
    return tensor_size(x, reduction_axes=x.axes.batch_axes())


def mean(x, reduction_axes=None, out_axes=None):
    # op_graph.py:4252-4266
    return sum(x, reduction_axes=reduction_axes, out_axes=out_axes) / \
        tensor_size(x, reduction_axes=reduction_axes, out_axes=out_axes)


def squared_L2(x, out_axes=None, reduction_axes=None):
    if reduction_axes is None and out_axes is None:
        reduction_axes = x.axes.sample_axes()
    return sum(x * x, out_axes=out_axes, reduction_axes=reduction_axes)


class OneHotOp(TensorOp):
    """Class indices -> one-hot along a new leading axis (op_graph.py:4107-4164)."""

    def __init__(self, x, axis, **kwargs):
        x = as_op(x)
        self.axis = axis
        super(OneHotOp, self).__init__(args=(x,), axes=make_axes((axis,)) + x.axes, **kwargs)


def one_hot(x, axis):
    return OneHotOp(x, axis)


class RngOp(TensorOp):
    """A tensor of x's axes filled with fresh random numbers at every execution; x itself is
    not read (op_graph.py:2786-2812)."""

    def __init__(self, distribution, params, x, **kwargs):
        if distribution not in ("uniform", "normal"):
            raise ValueError("unsupported distribution: {}".format(distribution))
        x = as_op(x)
        self.distribution = distribution
        self.params = params
        super(RngOp, self).__init__(args=(x,), axes=x.axes, **kwargs)


def uniform(x, low=0.0, high=1.0):
    """Uniform numbers in [low, high) with the axes of x (op_graph.py:2843-2855)."""
    return RngOp(distribution="uniform", params=dict(low=low, high=high), x=x)


def normal(x, loc=0.0, scale=1.0):
    """Normal numbers around loc with standard deviation scale (op_graph.py:2858-2870)."""
    return RngOp(distribution="normal", params=dict(loc=loc, scale=scale), x=x)


class LookupTableOp(TensorOp):
    """Forward lookup: rows (lut_axis 0) or columns (lut_axis 1) of a 2-D table selected by a
    1-D index tensor (op_graph/lookuptable.py:55-115).  `axes` are the output axes; the one at
    position lut_axis must be the index axis, the other one the table's remaining axis."""

    def __init__(self, lut, idx, axes, update=True, pad_idx=None, **kwargs):
        lut, idx = as_op(lut), as_op(idx)
        axes = make_axes(axes)
        if len(lut.shape) != 2:
            raise ValueError("lookup table shape must be length 2, found {}".format(len(lut.shape)))
        if len(idx.shape) != 1:
            raise ValueError("index shape must be length 1, found {}".format(len(idx.shape)))
        if not (lut.axes[0] in axes or lut.axes[1] in axes):
            raise ValueError("Output axes must indicate which axis to do lookup.  None of the "
                             "output axes is from lookup table.  Found lut axes: {} Found output "
                             "axes: {}.".format(lut.axes, axes))
        if idx.axes[0] not in axes:
            raise ValueError("Output axes must index axes.  Found index axes: {} Found output "
                             "axes: {}.".format(idx.axes, axes))
        self.lut_axis = 0 if lut.axes[1] in axes else 1
        self.pad_idx = pad_idx
        self.update = update
        if axes[self.lut_axis] != idx.axes[0]:
            raise ValueError("Cannot transpose lut axes implicitly")
        super(LookupTableOp, self).__init__(args=(lut, idx), axes=axes, **kwargs)


def lookuptable(lut, idx, axes, update=True, pad_idx=None):
    """Look `idx` up in `lut`; `axes` are the output axes (op_graph/lookuptable.py:20-36)."""
    return LookupTableOp(lut, idx, axes=axes, update=update, pad_idx=pad_idx)


class UnmatchedAxesError(ValueError):
    """y and t of a cross entropy do not broadcast to matching axes."""


class SigmoidOp(ValueOp):
    """sigmoid as the composite reciprocal(exp(-x) + 1) (op_graph.py:4183-4202)."""

    def __init__(self, x, **kwargs):
        super(SigmoidOp, self).__init__(**kwargs)
        self.x = x
        self.value_tensor = reciprocal(exp(-x) + 1)
        self.value_tensor.deriv_handler = self

    def generate_adjoints(self, add_delta, adjoints, delta):
        # op_graph.py:4200-4202
        add_delta(adjoints, self.x, delta * self.value_tensor * (1.0 - self.value_tensor))


def sigmoid(x):
    return SigmoidOp(as_op(x)).value_tensor


def sigmoidAtomic(x):
    return SigmoidAtomicOp(x)


class SoftmaxOp(ValueOp):
    """softmax as exp(x - max x) / sum of the same (op_graph.py:3819-3846).  The
    composite is kept reachable from its value (`deriv_handler`) so that a cross
    entropy can use the shifted input and the normaliser directly."""

    def __init__(self, x, normalization_axes=None, **kwargs):
        super(SoftmaxOp, self).__init__(**kwargs)
        if normalization_axes is None:
            rec = x.axes.recurrent_axis()
            normalization_axes = x.axes.sample_axes() - (
                make_axes(rec) if rec is not None else make_axes(()))
        self.x = x - max(x, reduction_axes=normalization_axes)
        self.exps = exp(self.x)
        self.Z = sum(self.exps, reduction_axes=normalization_axes)
        self.value_tensor = self.exps * reciprocal(self.Z)
        self.value_tensor.deriv_handler = self
        self.normalization_axes = normalization_axes

    def generate_adjoints(self, add_delta, adjoints, delta):
        # op_graph.py:3832-3846
        z = delta * self.value_tensor
        zs = sum(z, reduction_axes=self.normalization_axes)
        add_delta(adjoints, self.x, z - zs * self.value_tensor)


class StackOp(SequentialOp):
    """Joins identically-axed tensors along a new axis inserted at `pos`: every argument is
    assigned, on the device, into its slice of a temporary that has the new axis first, and the
    result is that temporary with the axes in the requested order (op_graph.py:2567-2619)."""

    def __init__(self, x_list, axis, pos=0, **kwargs):
        super(StackOp, self).__init__(**kwargs)
        self.pos = pos
        self.x_list = tuple(as_op(arg) for arg in x_list)
        if axis.length != len(self.x_list):
            raise ValueError("Axis must have the same length as x_list")
        arg_axes = self.x_list[0].axes
        result_axes = arg_axes[:pos] + make_axes(axis) + arg_axes[pos:]
        storage_axes = make_axes((axis,) + tuple(arg_axes))
        self.storage = temporary(axes=storage_axes, dtype=self.x_list[0].dtype).named("stack")
        slices = [slice(None)] * len(arg_axes)
        self.ops = [assign(tensor_slice(self.storage, [i] + slices, axes=arg_axes), axes_with_order(arg, arg_axes))
                    for i, arg in enumerate(self.x_list)] + \
                   [axes_with_order(value_of(self.storage), result_axes)]
        self.value_tensor.deriv_handler = self

    def generate_adjoints(self, add_delta, adjoints, delta):
        s = [slice(None)] * len(self.storage.axes)
        delta = axes_with_order(delta, self.value_tensor.axes)
        for i, x in enumerate(self.x_list):
            s[self.pos] = i
            piece = tensor_slice(delta, tuple(s), axes=delta.axes[:self.pos] + delta.axes[self.pos + 1:])
            add_delta(adjoints, x, axes_with_order(piece, x.axes))


def stack(x_list, axis, pos=0):
    return StackOp(x_list, axis, pos).value_tensor


class ConcatOp(SequentialOp):
    """Concatenates tensors along one axis each (same name, lengths may differ; the other axes
    are common): assignments into windows of a temporary (op_graph.py:2636-2708)."""

    def __init__(self, x_list, axis_list, **kwargs):
        super(ConcatOp, self).__init__(**kwargs)
        self.x_list = tuple(as_op(arg) for arg in x_list)
        self.axis_list = list(axis_list)
        arg_axes = self.x_list[0].axes
        ax = self.axis_list[0]
        common_axes = arg_axes - make_axes(ax)
        for ii, x in enumerate(self.x_list):
            if len(x.axes - common_axes) > 1:
                raise RuntimeError("Tensor {} has more than 1 axis not in common with other tensors".format(ii))
        self.concat_axis = make_axis(builtins.sum(a.length for a in self.axis_list), name=ax.name)
        ind = arg_axes.index(ax)
        axes_0, axes_1 = arg_axes[:ind], arg_axes[ind + 1:]
        result_axes = axes_0 + make_axes(self.concat_axis) + axes_1
        self.storage_axes = make_axes([self.concat_axis] + list(axes_0) + list(axes_1))
        self.storage = temporary(axes=self.storage_axes, dtype=self.x_list[0].dtype).named("concat")
        slices = [slice(None)] * (len(self.storage_axes) - 1)
        ops, start = [], 0
        for x, a in zip(self.x_list, self.axis_list):
            piece_axes = make_axes([a] + list(self.storage_axes[1:]))
            window = tensor_slice(self.storage, [slice(start, start + a.length)] + slices, axes=piece_axes)
            ops.append(assign(window, axes_with_order(x, piece_axes)))
            start += a.length
        self.ops = ops + [axes_with_order(value_of(self.storage), result_axes)]
        self.value_tensor.deriv_handler = self

    def generate_adjoints(self, add_delta, adjoints, delta):
        slices = [slice(None)] * (len(self.storage_axes) - 1)
        storage_delta = axes_with_order(delta, self.storage_axes)
        start = 0
        for x, a in zip(self.x_list, self.axis_list):
            piece_axes = make_axes([a] + list(self.storage_axes[1:]))
            piece = tensor_slice(storage_delta, [slice(start, start + a.length)] + slices, axes=piece_axes)
            add_delta(adjoints, x, axes_with_order(piece, x.axes))
            start += a.length


def concat_along_axis(x_list, axis):
    """The tensors of x_list joined along `axis`, which each of them has (by name); axes ordered
    as in the first (op_graph.py:2711-2737)."""
    if len(x_list) < 1:
        return x_list
    x_list = [as_op(x) for x in x_list]
    return ConcatOp(x_list, [x.axes[x.axes.index(axis)] for x in x_list]).value_tensor


def softmax(x, normalization_axes=None, **kwargs):
    return SoftmaxOp(as_op(x), normalization_axes, **kwargs).value_tensor


def _check_cross_entropy_axes(y, t):
    if (not y.axes.is_sub_set(t.axes)) and (not y.axes.is_super_set(t.axes)):
        raise UnmatchedAxesError(
            "y and t must broadcast to matching axes: {} vs. {}".format(y.axes, t.axes))


def cross_entropy_multi(y, t, usebits=False, out_axes=None, enable_softmax_opt=True,
                        enable_diff_opt=True):
    """Cross entropy of the distributions y (model) and t (truth), summed over the
    sample axes that are not recurrent (op_graph.py:4318-4390).  When y is a
    softmax, -sum(x t) + log Z on the shifted input replaces -sum(t log y); this
    relies on sum(t) == 1, as the reference's shortcut does."""
    y, t = as_op(y), as_op(t)
    _check_cross_entropy_axes(y, t)
    if out_axes is None:
        rec = y.axes.recurrent_axis()
        index_axes = y.axes.sample_axes() - (make_axes(rec) if rec is not None else make_axes(()))
        out_axes = y.axes - index_axes
    handler = getattr(y, "deriv_handler", None)
    if enable_softmax_opt and isinstance(handler, SoftmaxOp):
        s = -sum(handler.x * t, out_axes=out_axes)
        value = minimum(s + log(handler.Z), safelog_cutoff)
        if enable_diff_opt:
            value.deriv_handler = _SoftmaxCrossEntropyAdjoint(handler, s)
    else:
        value = -sum(safelog(y) * t, out_axes=out_axes)
    if usebits:
        value = value * float(1.0 / np.log(2.0))
    return value


class _SoftmaxCrossEntropyAdjoint(object):
    """d/dx of -sum(x t) + log Z is -t + softmax(x) (op_graph.py:4363-4365)."""

    def __init__(self, softmax_op, s):
        self.softmax_op, self.s = softmax_op, s

    def generate_adjoints(self, add_delta, adjoints, delta):
        add_delta(adjoints, self.s, delta)
        add_delta(adjoints, self.softmax_op.x, self.softmax_op.value_tensor * delta)


class _SigmoidCrossEntropyAdjoint(object):
    """Binary cross entropy of a sigmoid: d/dx = (y - t), d/dt = x (op_graph.py:4425-4427)."""

    def __init__(self, sigmoid_op, y, t):
        self.sigmoid_op, self.y, self.t = sigmoid_op, y, t

    def generate_adjoints(self, add_delta, adjoints, delta):
        add_delta(adjoints, self.sigmoid_op.x, (self.y - self.t) * delta)
        add_delta(adjoints, self.t, self.sigmoid_op.x * delta)


def cross_entropy_binary_inner(y, t, enable_sig_opt=True, enable_diff_opt=True):
    """Per-element binary cross entropy -(t log y + (1 - t) log(1 - y))
    (op_graph.py:4392-4451).  When y is a sigmoid of x the equivalent
    (1 - t) max(x, -cutoff) - log y is built instead."""
    y, t = as_op(y), as_op(t)
    _check_cross_entropy_axes(y, t)
    handler = getattr(y, "deriv_handler", None)
    value = -(safelog(y) * t + safelog(1 - y) * (1 - t))
    if isinstance(handler, SigmoidOp):
        if enable_sig_opt:
            value = (1 - t) * maximum(handler.x, -safelog_cutoff) - safelog(y)
        if enable_diff_opt:
            value.deriv_handler = _SigmoidCrossEntropyAdjoint(handler, y, t)
    return value


def cross_entropy_binary(y, t, usebits=False, out_axes=None, enable_sig_opt=True,
                         enable_diff_opt=True):
    """Binary cross entropy summed over the sample axes (op_graph.py:4454-4478)."""
    result = sum(cross_entropy_binary_inner(y, t, enable_sig_opt=enable_sig_opt,
                                            enable_diff_opt=enable_diff_opt),
                 out_axes=out_axes)
    if usebits:
        result = result * float(1.0 / np.log(2.0))
    return result
