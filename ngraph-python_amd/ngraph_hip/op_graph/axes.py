"""Named axes and strided tensor descriptions.

A compact counterpart of ngraph/op_graph/axes.py for the subset of behaviour
the elementwise / reduction path observes:

* `Axis` equality is by NAME only; unnamed axes get `Axis_<n>`
  (axes.py:113-131, 202-203).
* `Axes` is an ordered, duplicate-free tuple with concatenation, ordered set
  difference / union / intersection (axes.py:576-634), `lengths`, `size`,
  and the role queries (`batch_axis` is the axis named "N", the recurrent
  axis the one named "REC", axes.py:145-166, 469-527).
* `FlattenedAxis` groups several axes into one dimension (axes.py:999-1086).
* `TensorDescription` is shape + strides + offset over a base buffer; views
  (broadcast, reorder, flatten, unflatten, slice, cast, transpose) only
  rewrite those numbers (axes.py:1281-1620).  Strides are kept in ELEMENTS
  here (a flex tensor's storage item size differs from its logical dtype);
  `strides` reports bytes like the reference does.
"""
from __future__ import division
import collections.abc
import numbers

import numpy as np


def default_dtype(dtype=None):
    if dtype is None:
        dtype = np.dtype(np.float32)
    elif not isinstance(dtype, np.dtype) and not hasattr(dtype, "storage_bits"):
        dtype = np.dtype(dtype)
    return dtype


def default_int_dtype(dtype=None):
    if dtype is None:
        dtype = np.dtype(np.int32)
    elif not isinstance(dtype, np.dtype):
        dtype = np.dtype(dtype)
    return dtype


def make_axis(length=None, name=None, docstring=None):
    return Axis(length=length, name=name)


def make_axes(axes=()):
    return Axes(axes=axes)


class Axis(object):
    __name_counter = 0

    def __init__(self, length=None, name=None, **kwargs):
        assert "batch" not in kwargs and "recurrent" not in kwargs
        if name is None:
            name = "%s_%s" % (type(self).__name__, Axis.__name_counter)
            Axis.__name_counter += 1
        self.name = name
        if length is not None and length < 0:
            raise ValueError("Axis length {} must be >= 0".format(length))
        self.__length = length

    def named(self, name):
        self.name = name
        return self

    @property
    def is_flattened(self):
        return False

    @property
    def is_batch(self):
        return self.name == "N"

    @property
    def is_recurrent(self):
        return self.name == "REC"

    @property
    def is_channel(self):
        return self.name == "C"

    @property
    def length(self):
        return self.__length

    @length.setter
    def length(self, value):
        self.__length = value

    @property
    def axes(self):
        return Axes([self])

    def __repr__(self):
        return "Axis({name}: {length})".format(name=self.name, length=self.length)

    __str__ = __repr__

    def __eq__(self, other):
        return isinstance(other, Axis) and self.name == other.name

    def __ne__(self, other):
        return not self == other

    def __len__(self):
        return self.length

    def __add__(self, other):
        return Axes([self]) + other

    def __or__(self, other):
        return Axes([self]) | other

    def __and__(self, other):
        return Axes([self]) & other

    def __hash__(self):
        return hash(self.name)


def _sliced_length(s, incoming_length):
    start, stop, step = s.indices(incoming_length)
    if step is None:
        step = 1
    if (step > 0 and stop <= start) or (step < 0 and stop >= start):
        return 0
    return (abs(stop - start) + abs(step) - 1) // abs(step)


def slice_axis(axis, s):
    """Axis of the right length for axis[s]; keeps the name when the length is unchanged."""
    if s.step not in (None, 1, -1):
        raise ValueError("slice step {} not supported".format(s.step))
    new_length = len(range(axis.length)[s])
    if new_length == axis.length:
        return axis
    return make_axis(length=new_length, name=axis.name)


def duplicates(arr):
    seen, dups = set(), []
    for x in arr:
        key = x.name if isinstance(x, Axis) else x
        if key in seen:
            dups.append(key)
        seen.add(key)
    return dups


class Axes(object):
    def __init__(self, axes=None):
        if axes is None:
            axes = []
        elif isinstance(axes, Axis):
            axes = [axes]
        elif isinstance(axes, Axes):
            axes = tuple(axes)
        elif isinstance(axes, dict):
            axes = tuple(make_axis(length=v, name=k) for k, v in axes.items())
        else:
            axes = tuple(axes)

        def convert(seq):
            elems = []
            for x in seq:
                if isinstance(x, collections.abc.Iterable) and not isinstance(x, Axis):
                    x = Axes(convert(x)).flatten(force=True)
                elems.append(x)
            return elems

        axes = convert(axes)
        for x in axes:
            if not isinstance(x, Axis):
                raise ValueError("tried to initialize an Axes with object type {}. all values "
                                 "should be an instance of a type which inherits from Axis."
                                 .format(type(x)))
        if duplicates(axes):
            raise ValueError("The axes labels of a tensor cannot contain duplicates.  Found: {}"
                             .format(str(duplicates(axes))))
        self._axes = tuple(axes)

    @property
    def full_lengths(self):
        return tuple(a.axes.full_lengths if a.is_flattened else a.length for a in self)

    @property
    def names(self):
        return tuple(a.name for a in self)

    @property
    def lengths(self):
        return tuple(a.length for a in self)

    def batch_axes(self):
        return Axes(a for a in self if a.is_batch)

    def batch_axis(self):
        for a in self:
            if a.is_batch:
                return a
        return None

    def channel_axis(self):
        for a in self:
            if a.is_channel:
                return a
        return None

    def sample_axes(self):
        return Axes(a for a in self if not a.is_batch)

    def feature_axes(self):
        return Axes(a for a in self if not a.is_batch and not a.is_recurrent)

    def recurrent_axis(self):
        for a in self:
            if a.is_recurrent:
                return a
        return None

    def flatten(self, force=False):
        if not force and len(self) == 1:
            return self[0]
        return FlattenedAxis(self)

    def find_by_name(self, name):
        return Axes(a for a in self if a.name == name)

    def __iter__(self):
        return iter(self._axes)

    def __len__(self):
        return len(self._axes)

    def __getitem__(self, item):
        if isinstance(item, slice):
            return Axes(self._axes[item])
        return self._axes[item]

    def __add__(self, other):
        other = make_axes(other)
        common = self & other
        if len(common) != 0:
            raise ValueError("Trying to concatenate %s with %s, but they have common axes %s, "
                             "which is not allowed." % (self, other, common))
        return make_axes(tuple(self) + tuple(other))

    def __sub__(self, other):
        other = make_axes(other)
        return make_axes(a for a in self if a not in other)

    def __or__(self, other):
        other = make_axes(other)
        return make_axes(tuple(self) + tuple(a for a in other if a not in self))

    def __and__(self, other):
        other = make_axes(other)
        return make_axes(a for a in self._axes if a in other)

    def __eq__(self, other):
        if not isinstance(other, Axes):
            try:
                other = Axes(other)
            except (ValueError, TypeError):
                return False
        return self._axes.__eq__(other._axes)

    def __ne__(self, other):
        return not self == other

    def __bool__(self):
        return bool(self._axes)

    __nonzero__ = __bool__

    def __hash__(self):
        return hash(self._axes)

    def is_sub_set(self, other):
        return set(self.names).issubset(set(make_axes(other).names))

    def is_super_set(self, other):
        return set(self.names).issuperset(set(make_axes(other).names))

    def is_equal_set(self, other):
        return set(self.names) == set(make_axes(other).names)

    def is_not_equal_set(self, other):
        return not self.is_equal_set(other)

    @property
    def T(self):
        return Axes(reversed(self._axes))

    def index(self, axis):
        return self._axes.index(axis)

    @staticmethod
    def assert_valid_broadcast(axes, new_axes):
        removed = axes - new_axes
        if removed:
            raise ValueError("The new_axes of a broadcast operation must include all of the "
                             "axes from the origional set of axes. Missing: {}".format(removed))

    @property
    def size(self):
        return int(np.prod(self.lengths, dtype=np.int64)) if len(self) else 1

    def __repr__(self):
        return "Axes({})".format(", ".join(map(repr, self)))

    __str__ = __repr__

    @staticmethod
    def as_flattened_list(axes):
        out = []
        for a in axes:
            if a.is_flattened:
                out.extend(Axes.as_flattened_list(a.axes))
            else:
                out.append(a)
        return out


class FlattenedAxis(Axis):
    """Several axes viewed as one dimension (axes.py:999-1086)."""

    def __init__(self, axes, **kwargs):
        axes = Axes(axes)
        flat = []
        for a in axes:
            flat.extend(a.axes if a.is_flattened else [a])
        self._sub_axes = Axes(flat)
        length = int(np.prod([a.length for a in flat], dtype=np.int64)) if flat else 1
        name = kwargs.pop("name", None) or "Flattened_" + "_".join(a.name for a in flat)
        super(FlattenedAxis, self).__init__(length=length, name=name)

    @property
    def is_flattened(self):
        return True

    @property
    def is_batch(self):
        return any(a.is_batch for a in self._sub_axes)

    @property
    def empty(self):
        return len(self._sub_axes) == 0

    @property
    def single(self):
        return len(self._sub_axes) == 1

    @property
    def axes(self):
        return self._sub_axes

    def __eq__(self, other):
        return isinstance(other, FlattenedAxis) and self.axes == other.axes

    def __hash__(self):
        return hash(self.axes)

    def __repr__(self):
        return "FlattenedAxis({})".format(", ".join(repr(a) for a in self.axes))


class TensorDescription(object):
    """Shape, element strides and offset of a (view of a) buffer.

    `base` is the description that owns the buffer; a base has itself as base.
    """

    _counter = 0

    def __init__(self, axes, base=None, dtype=None, full_strides=None, offset=0,
                 is_persistent=False, is_input=False, is_placeholder=False, op=None, name=None):
        self.axes = Axes(axes)
        for axis in self.axes:
            if axis.length is None:
                raise ValueError("axes used in the constructor of TensorDescription must always "
                                 "have non-None length.  Axis {} has length None.".format(axis))
        self.__base = base
        self.dtype = default_dtype(dtype)
        self.offset = int(offset)                     # in elements
        self.ndim = len(self.axes)
        if full_strides is None:
            strides, acc = [], 1
            for axis in reversed(self.axes):
                strides.insert(0, acc)
                acc *= axis.length
            full_strides = strides
        self.full_strides = tuple(int(s) for s in full_strides)   # in elements
        assert len(self.full_strides) == self.ndim
        self.__is_persistent = is_persistent
        self.__is_input = is_input
        self.__is_placeholder = is_placeholder
        self.op = op
        if name is None:
            name = "td_%d" % TensorDescription._counter
            TensorDescription._counter += 1
        self.name = name

    def __repr__(self):
        return "TensorDescription({}, shape={}, strides={}, offset={})".format(
            self.base.name, self.shape, self.full_strides, self.offset)

    # -- flags inherited from the base ----------------------------------------
    @property
    def base(self):
        return self.__base or self

    def is_base(self):
        return self.__base is None

    @property
    def is_persistent(self):
        return self.base.__is_persistent if self.__base else self.__is_persistent

    @property
    def is_input(self):
        return self.base.__is_input if self.__base else self.__is_input

    @property
    def is_placeholder(self):
        return self.base.__is_placeholder if self.__base else self.__is_placeholder

    @property
    def parameter_key(self):
        return (self.shape, self.dtype if isinstance(self.dtype, np.dtype) else "flex",
                self.offset, self.full_strides)

    # -- geometry ----------------------------------------------------------------
    @property
    def shape(self):
        return self.axes.lengths

    @property
    def element_strides(self):
        return self.full_strides

    @property
    def itemsize(self):
        return self.dtype.itemsize

    @property
    def strides(self):
        return tuple(s * self.itemsize for s in self.full_strides)

    @property
    def sizes(self):
        return self.axes.lengths

    @property
    def tensor_size(self):
        """Bytes of the buffer a base description owns."""
        return self.axes.size * self.itemsize

    @property
    def c_contiguous(self):
        acc = 1
        for length, stride in zip(reversed(self.shape), reversed(self.full_strides)):
            if length != 1 and stride != acc:
                return False
            acc *= length
        return True

    @property
    def is_scalar_broadcast(self):
        return all(s == 0 or n == 1 for s, n in zip(self.full_strides, self.shape))

    def _view(self, axes, strides, offset=None):
        return TensorDescription(axes, base=self.base, dtype=self.dtype, full_strides=strides,
                                 offset=self.offset if offset is None else offset, op=self.op)

    # -- views -------------------------------------------------------------------
    def broadcast(self, new_axes):
        """View with `new_axes`; axes absent from this description get stride 0 (axes.py:1444-1457)."""
        Axes.assert_valid_broadcast(self.axes, new_axes)
        return self.reorder_and_broadcast(new_axes)

    def reorder(self, new_axes):
        new_axes = Axes(new_axes)
        if not self.axes.is_equal_set(new_axes):
            raise ValueError("Reorder can't change which axes are available, only the order. "
                             "{} and {} are different sets, not just order.".format(self, new_axes))
        return self.reorder_and_broadcast(new_axes)

    def reorder_and_broadcast(self, new_axes):
        new_axes = Axes(new_axes)
        strides = []
        for axis in new_axes:
            if axis in self.axes:
                strides.append(self.full_strides[self.axes.index(axis)])
            elif axis.is_flattened and all(a in self.axes for a in axis.axes) and len(axis.axes):
                sub = self._flatten_group(axis.axes)
                if sub is None:
                    raise ValueError("axes {} are not mergeable in this view".format(axis.axes))
                strides.append(sub)
            else:
                strides.append(0)
        return self._view(new_axes, strides)

    def _flatten_group(self, group):
        """Stride of the single dimension covering `group`, or None when not mergeable."""
        dims = [(a.length, self.full_strides[self.axes.index(a)]) for a in group]
        dims = [(n, s) for n, s in dims if n != 1]
        if not dims:
            return 0
        for (n0, s0), (n1, s1) in zip(dims[:-1], dims[1:]):
            if s0 != s1 * n1:
                return None
        return dims[-1][1]

    def can_flatten(self, new_axes):
        for axis in Axes(new_axes):
            if axis.is_flattened and self._flatten_group(axis.axes) is None:
                return False
        return True

    def flatten(self, new_axes):
        """View whose FlattenedAxis entries merge runs of this description's axes (axes.py:1281-1321)."""
        new_axes = Axes(new_axes)
        strides = []
        for axis in new_axes:
            if axis.is_flattened:
                s = self._flatten_group(axis.axes)
                if s is None:
                    raise ValueError("cannot flatten {} as a view; make it contiguous first"
                                     .format(axis))
                strides.append(s)
            else:
                strides.append(self.full_strides[self.axes.index(axis)])
        return self._view(new_axes, strides)

    def unflatten(self, new_axes):
        """Inverse of flatten: split every FlattenedAxis of this description (axes.py:1323-1403)."""
        new_axes = Axes(new_axes)
        strides = []
        for axis in self.axes:
            stride = self.full_strides[self.axes.index(axis)]
            if axis.is_flattened:
                acc, sub = 1, []
                for a in reversed(axis.axes):
                    sub.insert(0, stride * acc)
                    acc *= a.length
                strides.extend(sub)
            else:
                strides.append(stride)
        flat = []
        for axis in self.axes:
            flat.extend(axis.axes if axis.is_flattened else [axis])
        if Axes(flat) != new_axes:
            raise ValueError("unflatten target {} does not match {}".format(new_axes, Axes(flat)))
        return self._view(new_axes, strides)

    def transpose(self):
        return self._view(self.axes.T, tuple(reversed(self.full_strides)))

    def cast(self, new_axes):
        new_axes = Axes(new_axes)
        if new_axes.lengths != self.axes.lengths:
            raise ValueError("cast_axes: lengths {} != {}".format(new_axes.lengths, self.axes.lengths))
        return self._view(new_axes, self.full_strides)

    def slice(self, slices, new_axes):
        """View of self[slices]; integer entries drop the axis (axes.py:1553-1623)."""
        slices = list(slices) + [slice(None)] * (self.ndim - len(slices))
        offset, strides = self.offset, []
        for s, stride, length in zip(slices, self.full_strides, self.shape):
            if isinstance(s, slice):
                start, stop, step = s.indices(length)
                if step != 1:
                    if step == -1:
                        raise ValueError("negative-step slices need a copy; not supported as a view")
                    raise ValueError("slice step {} not supported".format(step))
                offset += start * stride
                strides.append(stride)
            else:
                idx = int(s)
                if idx < 0:
                    idx += length
                offset += idx * stride
        return self._view(Axes(new_axes), strides, offset=offset)

    def clone(self):
        return self._view(self.axes, self.full_strides)
